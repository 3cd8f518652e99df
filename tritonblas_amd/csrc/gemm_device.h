// Device side of the tile GEMM family for gfx950 (MI355X): LDS-staged operands, 16x16 MFMA tiles,
// fused scale/bias/cast epilogue, and the four tile schedules (data-parallel, work-stealing queues,
// Stream-K with partial-tile fixup, grouped expert table).
//
// One kernel template covers every element type: operands are moved as 16-byte "chunks" along K,
// both operands sit K-major in LDS, and only the MFMA instruction and the chunk->lane assignment
// depend on the type.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace tb {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));

enum : int { DT_F16 = 0, DT_BF16 = 1, DT_FP8 = 2, DT_FP4 = 3, DT_F32 = 4, DT_I8 = 5, DT_E5M2 = 6,
             DT_E4E5 = 7,    // A in e4m3, B in e5m2 (operand types only; never an output type)
             DT_E5E4 = 8 };  // A in e5m2, B in e4m3
// the two 8-bit float formats (OCP e4m3 = DT_FP8, e5m2) and their two mixtures share everything but the
// MFMA's format fields (0 = e4m3, 1 = e5m2, one field per operand)
constexpr bool is_f8(int dt) { return dt == DT_FP8 || dt == DT_E5M2 || dt == DT_E4E5 || dt == DT_E5E4; }
constexpr int f8_fmt_a(int dt) { return (dt == DT_E5M2 || dt == DT_E5E4) ? 1 : 0; }
constexpr int f8_fmt_b(int dt) { return (dt == DT_E5M2 || dt == DT_E4E5) ? 1 : 0; }
enum : int { MODE_STATIC = 0, MODE_WS = 1, MODE_SK = 2, MODE_GROUPED = 3 };
enum : int { WS_QUEUES = 0, WS_GLOBAL = 1, WS_HIERARCHICAL = 2 };   // how work-stealing workgroups find tiles
enum : int { LAY_K = 0, LAY_M = 1 };  // which index is contiguous in global memory for an operand

// Word offsets inside the control block at the head of a workspace.
enum : int { CTL_STATUS = 0, CTL_DONE = 1, CTL_EPOCH = 2, CTL_WORDS = 64 };
constexpr uint32_t EPOCH_ON_DEVICE = 0xFFFFFFFFu;   // GemmParams::epoch: the workspace's own count tags the launch
constexpr int COUNTER_STRIDE = 64;  // ints between queue counters: one 256-byte line each

// Measurement hooks of the K loop (skip the copies or the MFMAs; results are then meaningless) exist
// only in builds with -DTB_LAB_HOOKS; a shipped kernel cannot be told to skip work.
#ifdef TB_LAB_HOOKS
#define TB_LAB(p, bit) (((p).debug & (bit)) != 0)
#else
#define TB_LAB(p, bit) false
#endif

struct GemmParams {
  const uint8_t* A;
  const uint8_t* B;
  uint8_t* C;
  const float* sa;
  const float* sb;
  const uint8_t* bias;
  const uint8_t* mxa;
  const uint8_t* mxb;
  int32_t M, N;
  int64_t KU;                    // K extent in storage units (elements; bytes for packed fp4)
  int64_t a_sr, a_sk;            // strides in storage units: row (m) and k
  int64_t b_sr, b_sk;            // row (n) and k
  int64_t c_sm, c_sn;            // elements
  int64_t mxa_sr, mxa_sk, mxb_sr, mxb_sk;  // bytes
  int64_t bias_stride;
  int32_t c_type, bias_type;
  int32_t a_vec, b_vec, c_vec;   // 16-byte vector access is legal for this operand (c_vec: 4-element rows)
  int32_t c_line;                // C rows are 16-byte aligned with unit column stride: full-line store path
  int32_t c_nt;                  // C is larger than the L2s together: store it non-temporal so that it
                                 // does not push operand strips out of them
  int32_t mx_vec;                // scale rows can be read KSUB bytes at a time
  int32_t mx_lds;                // scale rows are 16-byte aligned and K/32 is a multiple of 32: stage scales in LDS
  int32_t tiles_m, tiles_n, total_tiles, k_iters;
  int32_t group_m, num_xcds, chunk;
  int32_t panel_n;               // tile order: column panels of this many tiles, swept top to bottom (0: one panel)
  int32_t mode;
  int32_t debug;                 // measurement builds only (TB_LAB_HOOKS): bit0 skip global->LDS copies, bit1 skip MFMA work
  // Stream-K
  int32_t sk_tiles;
  int32_t sk_unit;               // K steps per unit of the Stream-K split (0 or 1: single steps; the 4-wave kernels run K in
                                 // blocks of four steps, so their ranges are cut at multiples of four)
  int32_t sk_ws;                 // 1: the whole tiles in front of the Stream-K tail are drawn from the work-stealing queues
  float* P;
  uint32_t* flags;
  uint32_t epoch, spin_limit;
  uint32_t* ctl;
  // work stealing
  int32_t* counters;
  int32_t counters_per_xcd;
  const int32_t* cu_mask;
  int32_t ws_mode;               // WS_*
  int32_t ws_local, ws_global;   // hierarchical: tiles per XCD-local queue, tiles in the shared pool behind them
  // grouped
  const int32_t* group_offsets;
  int32_t num_groups;
  int64_t b_group_stride;   // storage units between consecutive experts' weights
  int64_t sb_group_stride;  // floats
  // grouped, two launches: phase 1 tiles every expert's rows with grp_big-row blocks but leaves a last
  // partial block of at most grp_thr rows to phase 2, which tiles just those rows with a short tile
  // (a handful of rows would otherwise cost a whole tall tile per column block).  Phase 0: one launch.
  // With grp_auto every workgroup of both launches first prices the two plans from the row counts
  // (rounds of tall tiles cost 4, rounds of short tiles 3) and both launches act on the same verdict:
  // either the first runs the one-launch table and the second does nothing, or they split the rows.
  int32_t grp_phase, grp_big, grp_thr;
  int32_t grp_auto, grp_small_bm;
  int32_t grp_other_tn, grp_other_grid;   // column tiles and grid of the other launch
  // grouped with a Stream-K tail (4-wave kernels): the tiles that do not fill whole rounds of the grid are cut into
  // K ranges as in MODE_SK; how many that is follows from the row counts, so every workgroup works it out
  // itself (sk_tail_tiles).  grp_sk_fix: what one extra piece of a tile costs its owner, in K steps.
  int32_t grp_sk, grp_sk_fix;
};

struct TileCtx {
  int m0, n0, m_lim, n_lim;
  const uint8_t* B;
  const float* sb;
};

template <int DT_, int BM_, int BN_, int BKB_, int WM_, int WN_, int ALAY_, int BLAY_, int MINB_ = 1,
          bool FAST_ = true, int STAGES_ = 2, bool USE_DMA_ = true>
struct Tile {
  static constexpr int DT = DT_, BM = BM_, BN = BN_, BKB = BKB_, WM = WM_, WN = WN_;
  static constexpr int ALAY = ALAY_, BLAY = BLAY_, MINB = MINB_, STAGES = STAGES_;
  // FAST: operands are 16-byte aligned, unit stride along their contiguous index, K is a multiple
  // of the K step (and row counts of M-contiguous operands multiples of 8): loaders carry no
  // bounds handling besides clamping rows.  !FAST: element-wise gathers, any strides, any K.
  static constexpr bool FAST = FAST_;
  static constexpr bool DMA = USE_DMA_ && FAST && ALAY == LAY_K && BLAY == LAY_K;  // global -> LDS without registers
  static constexpr int THREADS = WM * WN * 64;
  static constexpr int USZ = (DT == DT_F16 || DT == DT_BF16) ? 2 : (DT == DT_F32 ? 4 : 1);  // bytes per storage unit
  static constexpr int UPC = 16 / USZ;                                 // units per 16-byte chunk
  static constexpr int CPR = BKB / 16;                                 // chunks per tile row
  static constexpr int UPS = CPR * UPC;                                // units per K step
  static constexpr int EPU = (DT == DT_FP4) ? 2 : 1;                   // elements per unit
  static constexpr int BK = UPS * EPU;                                 // elements per K step
  static constexpr int KS = is_f8(DT) ? 8 : 4;                         // chunks one MFMA consumes per row
  static constexpr int KSUB = CPR / KS;                                // MFMA k-slices per K step
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int TM = WTM / 16, TN = WTN / 16;
  static constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  // MX scales (fp4, LDS-direct kernels): 16 scale bytes per tile row are staged in LDS at a time,
  // i.e. the scales of SCG consecutive K steps (one 32-element block = one 16-byte chunk = one byte),
  // in two buffers: one is read while the other takes the next group.
  static constexpr int SC_GB = 16;
  static constexpr int SCG = (DT == DT_FP4) ? SC_GB / CPR : 1;
  static constexpr int SC_BUF = (BM + BN) * SC_GB;
  static constexpr int SC_BYTES = (DT == DT_FP4 && DMA) ? 2 * SC_BUF : 0;
  static constexpr int LDS_TOTAL = LDS_BYTES + SC_BYTES;
  static constexpr int LDS_LIMIT = 160 * 1024;
  // the one word the schedules broadcast through LDS lives in the tile buffer's last 16 bytes when
  // the buffer takes the whole LDS (it is only used between K loops)
  static constexpr bool BCAST_IN_TILE = LDS_TOTAL + 16 > LDS_LIMIT;
  static constexpr int LDS_ALLOC = BCAST_IN_TILE ? LDS_TOTAL : LDS_TOTAL + 16;
  static_assert(LDS_TOTAL <= LDS_LIMIT, "tile buffers exceed the LDS of a CU");
  static constexpr int SWM = (CPR >= 16) ? 16 : CPR;       // XOR-swizzle range of the chunk index
  static_assert(CPR % KS == 0, "K step must hold whole MFMA slices");
  static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be MFMA aligned");
  static_assert(DT != DT_FP4 || KSUB == 1 || KSUB == 2 || KSUB == 4, "fp4 scale packing");
  static_assert(STAGES == 2 || (DMA && STAGES <= 4), "deeper pipelines need the LDS-direct loader");
  static_assert((BM * CPR) % 64 == 0 && (BN * CPR) % 64 == 0, "whole waves per operand copy");
  // XOR mask applied to the chunk index of a row: the low row bits, with odd and even groups of SWM
  // rows offset by one so that the 16 rows one MFMA operand read touches spread over all banks.
  __device__ static __forceinline__ int swz(int row) {
    return (SWM < 16) ? (((row % SWM) ^ ((row / SWM) & 1)) % SWM) : (row % SWM);
  }
};

struct LaneInfo {
  int tid, lane, r, g, wm0, wn0;
};

// ------------------------------------------------------------------------------------------------
// integer tile-order functions (same arithmetic as the host-side schedule tests check)
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ int chiplet_transform_chunked(int pid, int num_wg, int num_xcds, int chunk) {
  int block = num_xcds * chunk;
  if (pid > (num_wg / block) * block) return pid;
  int local = pid / num_xcds;
  int chunk_idx = local / chunk, pos = local % chunk, xcd = pid % num_xcds;
  return chunk_idx * block + xcd * chunk + pos;
}

// pid -> position when workgroup ids are dealt round-robin to the XCDs: ids of one XCD become contiguous
__host__ __device__ __forceinline__ int chiplet_transform(int pid, int num_wg, int num_xcds) {
  int xcd = pid % num_xcds, pos = pid / num_xcds;
  int min_per = num_wg / num_xcds, extra = num_wg % num_xcds;
  return xcd * min_per + (xcd < extra ? xcd : extra) + pos;
}

// Work-stealing queues.  WS_QUEUES: queue (xcd, slot) owns a contiguous run of the tile list: the list
// is cut into num_xcds parts and every part into S slots.  WS_GLOBAL: one queue over all tiles, entry
// idx is tile chiplet_transform(idx).  WS_HIERARCHICAL: queue xcd owns tiles [xcd*local, (xcd+1)*local),
// queue num_xcds (the shared pool) the rest.  Returns the queue's first tile and length.
__host__ __device__ __forceinline__ void ws_queue_range(int mode, int queue, int total, int X, int S, int local, int& first, int& count) {
  if (mode == WS_GLOBAL) { first = 0; count = queue == 0 ? total : 0; return; }
  if (mode == WS_HIERARCHICAL) {
    if (queue < X) { first = queue * local; count = local; }
    else { first = X * local; count = queue == X ? total - X * local : 0; }
    if (count < 0) count = 0;
    return;
  }
  const int qx = queue / S, qs = queue % S;
  const int per_xcd = (total + X - 1) / X;
  const int xbase = qx * per_xcd;
  int xcnt = (xbase + per_xcd < total ? xbase + per_xcd : total) - xbase;
  if (xcnt < 0) xcnt = 0;
  const int per_slot = (xcnt + S - 1) / S;
  const int sbase = qs * per_slot;
  count = (sbase + per_slot < xcnt ? sbase + per_slot : xcnt) - sbase;
  if (count < 0) count = 0;
  first = xbase + sbase;
}
__host__ __device__ __forceinline__ int ws_queue_tile(int mode, int first, int idx, int total, int X) {
  return mode == WS_GLOBAL ? chiplet_transform(idx, total, X) : first + idx;
}

// Tile id -> (row block, column block).  Column panels of panel_n tiles (the last may be narrower) are
// visited one after the other; inside a panel, groups of group_m row blocks are swept left to right,
// rows fastest.  Consecutive ids therefore share A row strips and B column strips, and a panel's B
// strips are reused by every row group before the next panel starts.
__host__ __device__ __forceinline__ void tile_coords(int tile, int tiles_m, int tiles_n, int group_m, int panel_n, int& pm, int& pn) {
  int first_n = 0, width = tiles_n;
  if (panel_n > 0 && panel_n < tiles_n) {
    int per_panel = tiles_m * panel_n;
    int pi = tile / per_panel;
    first_n = pi * panel_n;
    width = (tiles_n - first_n < panel_n) ? tiles_n - first_n : panel_n;
    tile -= pi * per_panel;
  }
  int in_group = group_m * width;
  int gid = tile / in_group;
  int first = gid * group_m;
  int gsz = (tiles_m - first < group_m) ? tiles_m - first : group_m;
  int rem = tile % in_group;
  pm = first + rem % gsz;
  pn = first_n + rem / gsz;
}

// ------------------------------------------------------------------------------------------------
// global -> LDS operand movement
// ------------------------------------------------------------------------------------------------
template <class T>
__device__ __forceinline__ v4i gather_units(const uint8_t* rowp, int64_t ku, int64_t s_k, int64_t KU) {
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  if constexpr (T::USZ == 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      int64_t k = ku + u;
      w[u] = (k < KU) ? *(const uint32_t*)(rowp + k * s_k * 4) : 0u;
    }
  } else if constexpr (T::USZ == 2) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      int64_t k = ku + u;
      uint32_t v = (k < KU) ? (uint32_t)(*(const uint16_t*)(rowp + k * s_k * 2)) : 0u;
      w[u >> 1] |= v << (16 * (u & 1));
    }
  } else {
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      int64_t k = ku + u;
      uint32_t v = (k < KU) ? (uint32_t)rowp[k * s_k] : 0u;
      w[u >> 2] |= v << (8 * (u & 3));
    }
  }
  v4i out = {(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
  return out;
}

// LDS image of an operand tile: ROWS rows of CPR chunks; chunk c of row r sits at chunk slot
// r*CPR + (c ^ swz(r)).  Slot q is filled by thread q % THREADS in round q / THREADS, so a wave
// always fills 64 consecutive slots (what the LDS-direct load requires).
template <class T, int ROWS, int LAY>
struct Operand {
  static constexpr int CHUNKS = ROWS * T::CPR;
  static constexpr int NCH = (CHUNKS + T::THREADS - 1) / T::THREADS;  // slots per thread
  static constexpr int RG = ROWS / 8;                                  // 8-row groups (LAY_M)
  static constexpr int NBLK = RG * T::CPR;                             // 8x8 blocks (LAY_M)
  static constexpr int NBT = (NBLK + T::THREADS - 1) / T::THREADS;
  static constexpr bool TRANSPOSING = T::FAST && LAY == LAY_M;
  static constexpr int NREG = TRANSPOSING ? NBT * 8 : NCH;
  static constexpr int NOFF = TRANSPOSING ? NBT : NCH;
  static_assert(!TRANSPOSING || T::USZ == 2, "transposing loader is for 16-bit operands");

  struct St {
    const uint8_t* base;     // FAST: tile origin; else matrix origin
    uint32_t off[NOFF];      // FAST: per-slot byte offset from the K-step origin
    int64_t s_row, s_k;      // storage units
    int row0, row_lim;
  };

  __device__ static __forceinline__ void init(St& st, const uint8_t* mat, int64_t s_row, int64_t s_k, int row0,
                                              int row_lim, int tid) {
    st.s_row = s_row; st.s_k = s_k; st.row0 = row0; st.row_lim = row_lim;
    const int rows_valid = row_lim - row0;
    if constexpr (!T::FAST) {
      st.base = mat;
    } else if constexpr (LAY == LAY_K) {
      st.base = mat + (int64_t)row0 * s_row * T::USZ;
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        int q = i * T::THREADS + tid;
        int row = q / T::CPR, pc = q % T::CPR;
        int c = pc ^ T::swz(row);
        int rowc = min(row, rows_valid - 1);
        st.off[i] = (uint32_t)(rowc * (int)(s_row * T::USZ) + c * 16);
      }
    } else {
      st.base = mat + (int64_t)row0 * 2;
      const int last = ((rows_valid - 1) / 8) * 8;
#pragma unroll
      for (int ib = 0; ib < NBT; ++ib) {
        int b = ib * T::THREADS + tid;
        int rg = b % RG, c = b / RG;
        st.off[ib] = (uint32_t)(min(rg * 8, last) * 2 + c * 8 * (int)(s_k * 2));
      }
    }
  }

  // K-step origin for iteration `it`
  __device__ static __forceinline__ const uint8_t* step_ptr(const St& st, int it) {
    if constexpr (!T::FAST) return st.base;
    else if constexpr (LAY == LAY_K) return st.base + (int64_t)it * T::BKB;
    else return st.base + (int64_t)it * T::UPS * st.s_k * 2;
  }

  // LDS-direct copy of K step `it` into `lds` (no registers involved).  Written as inline assembly
  // for two reasons: the address is a scalar base plus a loop-invariant 32-bit lane offset, and the
  // compiler must not know that these vector-memory operations write LDS, otherwise it drains every
  // outstanding copy (vmcnt(0)) in front of the next LDS read and the software pipeline collapses.
  // Completion is tracked by hand with s_waitcnt vmcnt(N) before the barrier that publishes a stage.
  // s_nop 3: one wait state between the write of m0 and its use, and five between a scalar base that
  // the compiler may just have written with a vector instruction and the load that reads it.
  __device__ static __forceinline__ void dma(const St& st, int it, uint8_t* lds, int tid) {
    const uint8_t* gp = step_ptr(st, it);
    const int wave_slot = __builtin_amdgcn_readfirstlane(tid & ~63);
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      if (CHUNKS % T::THREADS != 0 && i * T::THREADS + wave_slot >= CHUNKS) continue;
      const uint32_t dst = lds0 + (uint32_t)((i * T::THREADS + wave_slot) * 16);
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tglobal_load_lds_dwordx4 %1, %2"
                   :
                   : "s"(dst), "v"(st.off[i]), "s"(gp)
                   : "memory", "m0");
    }
  }

  __device__ static __forceinline__ void gload(v4i (&r)[NREG], const St& st, int it, int64_t KU, int tid) {
    const uint8_t* gp = step_ptr(st, it);
    if constexpr (!T::FAST) {
      const int64_t ku0 = (int64_t)it * T::UPS;
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        int q = i * T::THREADS + tid;
        if (CHUNKS % T::THREADS != 0 && q >= CHUNKS) continue;
        int row = q / T::CPR, pc = q % T::CPR;
        int c = pc ^ T::swz(row);
        int64_t grow = min(st.row0 + row, st.row_lim - 1);
        r[i] = gather_units<T>(gp + grow * st.s_row * T::USZ, ku0 + (int64_t)c * T::UPC, st.s_k, KU);
      }
    } else if constexpr (LAY == LAY_K) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        if (CHUNKS % T::THREADS != 0 && i * T::THREADS + tid >= CHUNKS) continue;
        r[i] = *(const v4i*)(gp + st.off[i]);
      }
    } else {
      const int64_t ldk = st.s_k * 2;
#pragma unroll
      for (int ib = 0; ib < NBT; ++ib) {
        if (NBLK % T::THREADS != 0 && ib * T::THREADS + tid >= NBLK) continue;
        uint32_t w[8][4];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          v4i v = *(const v4i*)(gp + st.off[ib] + j * ldk);
          w[j][0] = v.x; w[j][1] = v.y; w[j][2] = v.z; w[j][3] = v.w;
        }
        // 8x8 transpose of 16-bit values: out row i, dword d holds k = 2d (low half) and 2d+1 (high).
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          uint32_t o[4];
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            uint32_t lo = w[2 * d][i >> 1], hi = w[2 * d + 1][i >> 1];
            o[d] = (i & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
          }
          v4i ov = {(int)o[0], (int)o[1], (int)o[2], (int)o[3]};
          r[ib * 8 + i] = ov;
        }
      }
    }
  }

  __device__ static __forceinline__ void sstore(uint8_t* lds, const v4i (&r)[NREG], int tid) {
    if constexpr (!TRANSPOSING) {
#pragma unroll
      for (int i = 0; i < NCH; ++i) {
        int q = i * T::THREADS + tid;
        if (CHUNKS % T::THREADS != 0 && q >= CHUNKS) continue;
        *(v4i*)(lds + q * 16) = r[i];
      }
    } else {
#pragma unroll
      for (int ib = 0; ib < NBT; ++ib) {
        int b = ib * T::THREADS + tid;
        if (NBLK % T::THREADS != 0 && b >= NBLK) continue;
        int rg = b % RG, c = b / RG;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          int row = rg * 8 + i;
          *(v4i*)(lds + row * T::BKB + ((c ^ T::swz(row)) << 4)) = r[ib * 8 + i];
        }
      }
    }
  }
};

// ------------------------------------------------------------------------------------------------
// LDS -> MFMA operand fragments
// ------------------------------------------------------------------------------------------------
template <class T>
struct Frag {
  using type = typename std::conditional<is_f8(T::DT), v8i, v4i>::type;

  // row: tile row of this lane (wave row base + 16*t + lane%16); g = lane/16; m = swizzle mask of row.
  __device__ static __forceinline__ type read(const uint8_t* lds, int row, int ks, int g, int m) {
    const uint8_t* rp = lds + row * T::BKB;
    if constexpr (is_f8(T::DT)) {
      int c0 = ks * 8 + 2 * g;
      v4i lo = *(const v4i*)(rp + ((c0 ^ m) << 4));
      v4i hi = *(const v4i*)(rp + (((c0 + 1) ^ m) << 4));
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    } else {
      // lane group g owns KSUB consecutive chunks.  fp4: their scale bytes are adjacent; all types:
      // the four groups of one read then sit KSUB chunks apart, which spreads a wave's 64 addresses
      // over the LDS banks (measured conflict-free, unlike groups reading four adjacent chunks).
      int c = g * T::KSUB + ks;
      return *(const v4i*)(rp + ((c ^ m) << 4));
    }
  }
};

// D(16x16) += X(16xk) * Y(16xk)^T; lane l holds D[4*(l/16)+j][l%16], j = 0..3.
template <class T, int KSI>
__device__ __forceinline__ v4f mma(typename Frag<T>::type x, typename Frag<T>::type y, v4f c, uint32_t sx, uint32_t sy) {
  if constexpr (T::DT == DT_F16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, x), __builtin_bit_cast(h8, y), c, 0, 0, 0);
  } else if constexpr (T::DT == DT_BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, x), __builtin_bit_cast(bf8, y), c, 0, 0, 0);
  } else if constexpr (T::DT == DT_F32) {
    // four 16x16x4 steps: lane group g feeds k = 4g + i to step i (any assignment works as long as
    // both operands use the same one), so one 16-byte fragment is consumed without shuffles
    // (reinterpret the whole vectors: a bit cast of one vector *element* reads element 0 with this compiler)
    const v4f xf = __builtin_bit_cast(v4f, x), yf = __builtin_bit_cast(v4f, y);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(xf[0], yf[0], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(xf[1], yf[1], c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_16x16x4f32(xf[2], yf[2], c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x4f32(xf[3], yf[3], c, 0, 0, 0);
  } else if constexpr (T::DT == DT_I8) {
    // exact int32 sums: the accumulator registers hold integers until the K loop ends
    return __builtin_bit_cast(v4f, __builtin_amdgcn_mfma_i32_16x16x64_i8(x, y, __builtin_bit_cast(v4i, c), 0, 0, 0));
  } else if constexpr (is_f8(T::DT)) {
    // (x is the B fragment, y the A fragment: the first format field is B's)
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x, y, c, f8_fmt_b(T::DT), f8_fmt_a(T::DT), 0, 0, 0, 0);
  } else {
    v8i x8 = {x.x, x.y, x.z, x.w, 0, 0, 0, 0};
    v8i y8 = {y.x, y.y, y.z, y.w, 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x8, y8, c, 4, 4, KSI, sx, KSI, sy);
  }
}

// E8M0 scale bytes of one lane for one K step: KSUB consecutive 32-blocks starting at kb, packed
// little-endian into a dword; blocks at or past kb_total read as 127 (= 1.0) so that zero-filled
// data cannot meet a NaN scale.
template <class T>
__device__ __forceinline__ uint32_t load_mx(const uint8_t* rowp, int64_t s_k, int64_t kb, int64_t kb_total, bool vec) {
  if (vec && kb + T::KSUB <= kb_total) {
    if constexpr (T::KSUB == 4) return *(const uint32_t*)(rowp + kb);
    if constexpr (T::KSUB == 2) return *(const uint16_t*)(rowp + kb);
    if constexpr (T::KSUB == 1) return *(rowp + kb);
  }
  uint32_t w = 0;
#pragma unroll
  for (int j = 0; j < T::KSUB; ++j) {
    uint32_t v = (kb + j < kb_total) ? (uint32_t)rowp[(kb + j) * s_k] : 127u;
    w |= v << (8 * j);
  }
  return w;
}

__device__ __forceinline__ void wait_vm0() { __builtin_amdgcn_s_waitcnt(0x0F70); }  // vmcnt(0) only

// ------------------------------------------------------------------------------------------------
// K loop: accumulates k iterations [it0, it1) of one output tile
// ------------------------------------------------------------------------------------------------
// WHOLE: the caller only ever passes complete tiles (it0 = 0, it1 = k_iters).
template <class T, bool WHOLE>
__device__ __forceinline__ void mainloop(const GemmParams& p, const TileCtx& tc, int it0, int it1,
                                         v4f (&acc)[T::TM][T::TN], uint8_t* lds, const LaneInfo& li) {
  using OA = Operand<T, T::BM, T::ALAY>;
  using OB = Operand<T, T::BN, T::BLAY>;
  using frag_t = typename Frag<T>::type;
  typename OA::St sa;
  typename OB::St sb;
  OA::init(sa, p.A, p.a_sr, p.a_sk, tc.m0, tc.m_lim, li.tid);
  OB::init(sb, tc.B, p.b_sr, p.b_sk, tc.n0, tc.n_lim, li.tid);
  uint32_t sca[T::TM], scb[T::TN], nsca[T::TM], nscb[T::TN];
  const int swm = T::swz(li.r);
  const int64_t kb_total = (p.KU * T::EPU) / 32;

#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < T::TM; ++i) sca[i] = nsca[i] = 0;
#pragma unroll
  for (int j = 0; j < T::TN; ++j) scb[j] = nscb[j] = 0;

  auto load_scales = [&](int it, uint32_t(&xa)[T::TM], uint32_t(&xb)[T::TN]) {
    if constexpr (T::DT == DT_FP4) {
      int64_t kb = (int64_t)it * T::CPR + li.g * T::KSUB;
#pragma unroll
      for (int i = 0; i < T::TM; ++i) {
        int64_t row = min(tc.m0 + li.wm0 + i * 16 + li.r, tc.m_lim - 1);
        xa[i] = load_mx<T>(p.mxa + row * p.mxa_sr, p.mxa_sk, kb, kb_total, p.mx_vec);
      }
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        int64_t row = min(tc.n0 + li.wn0 + j * 16 + li.r, tc.n_lim - 1);
        xb[j] = load_mx<T>(p.mxb + row * p.mxb_sr, p.mxb_sk, kb, kb_total, p.mx_vec);
      }
    }
  };

  constexpr bool MXG = (T::DT == DT_FP4) && T::DMA;   // MX scales staged through LDS

  // One K step of MFMAs from an LDS stage.  The A-side fragment of row block i+1 is requested before
  // the MFMAs of row block i are issued, so an LDS read is always in flight under the matrix pipe.
  auto compute = [&](const uint8_t* sA, const uint8_t* sB) {
#pragma unroll
    for (int ks = 0; ks < T::KSUB; ++ks) {
      frag_t bf[T::TN];
#pragma unroll
      for (int j = 0; j < T::TN; ++j) bf[j] = Frag<T>::read(sB, li.wn0 + j * 16 + li.r, ks, li.g, swm);
      frag_t af[2];
      af[0] = Frag<T>::read(sA, li.wm0 + li.r, ks, li.g, swm);
#pragma unroll
      for (int i = 0; i < T::TM; ++i) {
        if (i + 1 < T::TM) af[(i + 1) & 1] = Frag<T>::read(sA, li.wm0 + (i + 1) * 16 + li.r, ks, li.g, swm);
#pragma unroll
        for (int j = 0; j < T::TN; ++j) {
          // output rows follow the first MFMA operand: feed B there so that one lane owns four
          // consecutive n of one m (contiguous in a row-major C).
#define TB_MMA(KS) \
  if (ks == KS) acc[i][j] = mma<T, KS>(bf[j], af[i & 1], acc[i][j], scb[j], sca[i]);
          TB_MMA(0) TB_MMA(1) TB_MMA(2) TB_MMA(3)
#undef TB_MMA
        }
      }
      // pin the issue order for the machine scheduler: B fragments and the first A fragment, then
      // alternately the next A fragment's reads and one row block of MFMAs
      constexpr int RPF = is_f8(T::DT) ? 2 : 1;  // LDS reads per fragment
      __builtin_amdgcn_sched_group_barrier(0x100, RPF * (T::TN + 1), 0);
#pragma unroll
      for (int i = 0; i + 1 < T::TM; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x100, RPF, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, T::TN, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, T::TN, 0);
    }
  };

  if constexpr (T::DMA) {
    constexpr int S = T::STAGES;
    // Stage (it - it0) % S holds K step `it`.  One "group" is what a wave issues per K step: its share
    // of both operand copies.  All S stages are filled up front; afterwards the copy of step it+S is
    // issued in the middle of step `it`, right after the barrier that frees that step's stage.
    constexpr int NG = OA::NCH + OB::NCH;
    static_assert((S - 1) * NG <= 63, "vmcnt range");

    // ---- MX scales (fp4).  A scale group = SC_GB scale bytes of every tile row = the scales of SCG
    // K steps; group g is copied raw into buffer g & 1: per row [step][lane group][KSUB bytes], so
    // the KSUB bytes a lane needs for one K step and row block are one small LDS read, straight
    // from the copy.  The scales of step it+1 are read during the last slice of step `it`: those of
    // row block i once its MFMAs are issued, the rest behind the barrier.  Group g is therefore
    // requested after the barrier of step g*SCG - 3 (everybody has then read the last scales of
    // group g-2) and has landed by the wait of step g*SCG - 2, whose barrier publishes it (the
    // scale copy is issued ahead of the operand copies of its step, and the wait of the next step
    // lets at most one step's operand copies stay in flight).
    uint8_t* sc_lds = lds + T::LDS_BYTES;
    constexpr int NQ = T::BM + T::BN;                               // one 16-byte chunk per row and group
    constexpr int NSCH = MXG ? (NQ + T::THREADS - 1) / T::THREADS : 1;
    static_assert(!MXG || T::SC_GB == 16, "one copy chunk per row");
    static_assert(!MXG || T::KSUB <= 2, "scale reads are one or two bytes");
    constexpr int SC_LEAD = 3;
    static_assert(!MXG || S <= 3, "with deeper pipelines the scale copy would land a step later");
    static_assert(!MXG || T::SCG + 1 >= SC_LEAD, "a scale buffer is free again before its next group is requested");
    const uint8_t* scp[NSCH];
    const int g0 = it0 / T::SCG;
    const uint8_t* sc_ra = sc_lds + (li.wm0 + li.r) * T::SC_GB + li.g * T::KSUB;
    const uint8_t* sc_rb = sc_lds + (T::BM + li.wn0 + li.r) * T::SC_GB + li.g * T::KSUB;
    if constexpr (MXG) {
#pragma unroll
      for (int i = 0; i < NSCH; ++i) {
        const int row = i * T::THREADS + li.tid;
        if (row < T::BM) scp[i] = p.mxa + (int64_t)min(tc.m0 + row, tc.m_lim - 1) * p.mxa_sr;
        else scp[i] = p.mxb + (int64_t)min(tc.n0 + row - T::BM, tc.n_lim - 1) * p.mxb_sr;
      }
    }
    auto sc_dma = [&](int grp) {
      if constexpr (MXG) {
        const int wave_slot = __builtin_amdgcn_readfirstlane(li.tid & ~63);
        const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)sc_lds) + (grp & 1) * T::SC_BUF;
#pragma unroll
        for (int i = 0; i < NSCH; ++i) {
          if (NQ % T::THREADS != 0 && i * T::THREADS + wave_slot >= NQ) continue;
          const uint32_t dst = lds0 + (uint32_t)((i * T::THREADS + wave_slot) * 16);
          const uint8_t* src = scp[i] + (int64_t)grp * T::SC_GB;
          asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(dst), "v"(src) : "memory", "m0");
        }
      }
    };
    // the scale bytes of K step `it`: sca for q < TM, scb behind
    auto sc_request = [&](int it, int q, uint32_t(&xa)[T::TM], uint32_t(&xb)[T::TN]) {
      if constexpr (MXG) {
        const int off = ((it / T::SCG) & 1) * T::SC_BUF + (it % T::SCG) * T::CPR;
        const uint8_t* src = (q < T::TM) ? sc_ra + off + q * 16 * T::SC_GB : sc_rb + off + (q - T::TM) * 16 * T::SC_GB;
        const uint32_t v = (T::KSUB == 2) ? (uint32_t)(*(const uint16_t*)src) : (uint32_t)(*src);
        if (q < T::TM) xa[q] = v; else xb[q - T::TM] = v;
      }
    };
    if constexpr (MXG) {
      sc_dma(g0);
      if ((g0 + 1) * T::SCG < it1) sc_dma(g0 + 1);
    }
    int issued = 0;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      if (it0 + s < it1) {
        OA::dma(sa, it0 + s, lds + s * T::STAGE_BYTES, li.tid);
        OB::dma(sb, it0 + s, lds + s * T::STAGE_BYTES + T::A_BYTES, li.tid);
        ++issued;
      }
    }
    // step it0 must have landed; the younger stages may stay in flight (vmcnt counts in issue order)
    if (issued == S) __builtin_amdgcn_s_waitcnt(0x0F70 | (((S - 1) * NG) & 0xF) | ((((S - 1) * NG) >> 4) << 14));
    else wait_vm0();
    __syncthreads();
    if constexpr (MXG) {
#pragma unroll
      for (int q = 0; q < T::TM + T::TN; ++q) sc_request(it0, q, sca, scb);
    }

    // ---- software pipeline over (K step, MFMA slice) blocks ------------------------------------
    // On entry to a block its B fragments and its first A fragment are already in registers: they
    // were requested under the last row block of MFMAs of the block before.  Inside a block the A
    // fragment of row block i+1 is requested before the MFMAs of row block i.  The barrier that ends
    // a K step therefore sits in front of the last row block of its last slice, whose operands are
    // in registers: after it the freed stage is refilled, the next step's fragments are requested,
    // and the matrix pipe has that row block to chew on while they arrive.
    frag_t bf[T::TN];
    frag_t afn;
    auto request_b = [&](const uint8_t* sB, int ks, int j) { bf[j] = Frag<T>::read(sB, li.wn0 + j * 16 + li.r, ks, li.g, swm); };
    auto request_a = [&](const uint8_t* sA, int ks, int i) { return Frag<T>::read(sA, li.wm0 + i * 16 + li.r, ks, li.g, swm); };
    constexpr int RPF = is_f8(T::DT) ? 2 : 1;  // LDS reads per fragment

    // one block: slice KSV of the K step in stage (sA, sB).  `boundary` runs before the last row block;
    // afterwards the fragments of slice nks of stage (nA, nB) are requested.  After the last step of
    // the range that request still runs (no branch in the pipeline): it reads whatever the next stage
    // holds and nobody uses the result.
    auto block = [&](auto KSC, const uint8_t* sA, auto&& boundary, const uint8_t* nA, const uint8_t* nB, int nks, int nit) {
      constexpr int KSV = decltype(KSC)::value;
      constexpr bool LAST = MXG && KSV + 1 == T::KSUB;   // the next block belongs to K step nit: fetch its scales
      frag_t af[2];
      af[0] = afn;
#pragma unroll
      for (int i = 0; i < T::TM; ++i) {
        if constexpr (LAST) { if (i >= 1) sc_request(nit, i - 1, nsca, nscb); }
        if (i + 1 < T::TM) af[(i + 1) & 1] = request_a(sA, KSV, i + 1);
        if (i + 1 == T::TM) {
          // pin the issue order so far for the machine scheduler (the barrier inside `boundary` ends
          // a scheduling region): one fragment request (plus a scale read), then one row block of MFMAs
#pragma unroll
          for (int q = 0; q + 1 < T::TM; ++q) {
            if (LAST && q >= 1) __builtin_amdgcn_sched_group_barrier(0x100, RPF + 1, 0);
            else __builtin_amdgcn_sched_group_barrier(0x100, RPF, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, T::TN, 0);
          }
          if constexpr (LAST) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            // instruction selection is free to place the (side-effect-free) MFMAs behind the
            // barrier; an empty statement that "uses" their results keeps them in front of it
#pragma unroll
            for (int q = 0; q + 1 < T::TM; ++q) {
              static_assert(!MXG || T::TN == 4 || T::TN == 2, "pin list");
              if constexpr (T::TN == 4) asm volatile("" : "+v"(acc[q][0]), "+v"(acc[q][1]), "+v"(acc[q][2]), "+v"(acc[q][3]));
              else asm volatile("" : "+v"(acc[q][0]), "+v"(acc[q][1]));
            }
          }
          boundary();
          afn = request_a(nA, nks, 0);
        }
#pragma unroll
        for (int j = 0; j < T::TN; ++j) {
          // output rows follow the first MFMA operand: feed B there so that one lane owns four
          // consecutive n of one m (contiguous in a row-major C).
          acc[i][j] = mma<T, MXG ? KSV : 0>(bf[j], af[i & 1], acc[i][j], scb[j], sca[i]);
          if (i + 1 == T::TM) {
            request_b(nB, nks, j);
            if constexpr (LAST) {
              if (j == 0) sc_request(nit, T::TM - 1, nsca, nscb);
              sc_request(nit, T::TM + j, nsca, nscb);
            }
          }
        }
      }
      // last row block: the next A fragment, then MFMAs and B fragment (and scale) requests alternate
      __builtin_amdgcn_sched_group_barrier(0x100, RPF, 0);
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (LAST && j == 0) __builtin_amdgcn_sched_group_barrier(0x100, RPF + 2, 0);
        else if (LAST) __builtin_amdgcn_sched_group_barrier(0x100, RPF + 1, 0);
        else __builtin_amdgcn_sched_group_barrier(0x100, RPF, 0);
      }
      if constexpr (MXG && !LAST) {
        // (same reason as above: keeps this slice's last row block in front of the next slice)
        if constexpr (T::TN == 4) asm volatile("" : "+v"(acc[T::TM - 1][0]), "+v"(acc[T::TM - 1][1]), "+v"(acc[T::TM - 1][2]), "+v"(acc[T::TM - 1][3]));
        else asm volatile("" : "+v"(acc[T::TM - 1][0]), "+v"(acc[T::TM - 1][1]));
      }
      if constexpr (LAST) {
#pragma unroll
        for (int i = 0; i < T::TM; ++i) sca[i] = nsca[i];
#pragma unroll
        for (int j = 0; j < T::TN; ++j) scb[j] = nscb[j];
      }
    };

    // fragments of the first block
#pragma unroll
    for (int j = 0; j < T::TN; ++j) request_b(lds + T::A_BYTES, 0, j);
    afn = request_a(lds, 0, 0);

    int stage = 0;
    auto kstep = [&](int it) {
      int nstage = (stage + 1 == S) ? 0 : stage + 1;
      const uint8_t* sA = lds + stage * T::STAGE_BYTES;
      const uint8_t* sB = sA + T::A_BYTES;
      const uint8_t* nA = lds + nstage * T::STAGE_BYTES;
      const uint8_t* nB = nA + T::A_BYTES;
      // end of the K step: step it+1 must have landed (the S-2 younger copies may stay in flight while
      // they all exist; near the end of the range drain fully), every wave must be done reading this
      // stage, then the stage takes the copy of step it+S
      auto boundary = [&]() {
        // (lgkmcnt(0): this wave's reads of the stage have returned before anyone may overwrite it)
        if (S > 2 && it + S - 1 < it1) {
          constexpr int ALLOWED = (S - 2) * NG;
          __builtin_amdgcn_s_waitcnt(0x0070 | (ALLOWED & 0xF) | ((ALLOWED >> 4) << 14));
        } else {
          __builtin_amdgcn_s_waitcnt(0x0070);
        }
        __syncthreads();
        if constexpr (MXG) {
          if ((it + SC_LEAD) % T::SCG == 0) {
            const int grp = (it + SC_LEAD) / T::SCG;
            if (grp >= g0 + 2 && grp * T::SCG < it1) sc_dma(grp);   // (older than the operand copies below)
          }
        }
        if (it + S < it1 && !TB_LAB(p, 1)) {
          OA::dma(sa, it + S, lds + stage * T::STAGE_BYTES, li.tid);
          OB::dma(sb, it + S, lds + stage * T::STAGE_BYTES + T::A_BYTES, li.tid);
        }
      };
      auto nothing = []() {};
      if (TB_LAB(p, 2)) {
        boundary();
      } else {
        if constexpr (T::KSUB == 1) {
          block(std::integral_constant<int, 0>{}, sA, boundary, nA, nB, 0, it + 1);
        } else if constexpr (T::KSUB == 2) {
          block(std::integral_constant<int, 0>{}, sA, nothing, sA, sB, 1, it);
          block(std::integral_constant<int, 1>{}, sA, boundary, nA, nB, 0, it + 1);
        } else {
          static_assert(T::KSUB == 4, "MFMA slices per K step");
          block(std::integral_constant<int, 0>{}, sA, nothing, sA, sB, 1, it);
          block(std::integral_constant<int, 1>{}, sA, nothing, sA, sB, 2, it);
          block(std::integral_constant<int, 2>{}, sA, nothing, sA, sB, 3, it);
          block(std::integral_constant<int, 3>{}, sA, boundary, nA, nB, 0, it + 1);
        }
      }
      stage = nstage;
    };
    for (int it = it0; it < it1; ++it) kstep(it);
  } else {
    v4i ra[OA::NREG], rb[OB::NREG];
    uint8_t* sA0 = lds;
    uint8_t* sB0 = lds + T::A_BYTES;
    OA::gload(ra, sa, it0, p.KU, li.tid);
    OB::gload(rb, sb, it0, p.KU, li.tid);
    load_scales(it0, sca, scb);
    OA::sstore(sA0, ra, li.tid);
    OB::sstore(sB0, rb, li.tid);
    __syncthreads();
    for (int it = it0; it < it1; ++it) {
      const int cur = (it - it0) & 1;
      const bool has_next = it + 1 < it1;
      if (has_next) {
        OA::gload(ra, sa, it + 1, p.KU, li.tid);
        OB::gload(rb, sb, it + 1, p.KU, li.tid);
        load_scales(it + 1, nsca, nscb);
      }
      if (!TB_LAB(p, 2)) compute(sA0 + cur * T::STAGE_BYTES, sB0 + cur * T::STAGE_BYTES);
      if (has_next) {
        OA::sstore(sA0 + (cur ^ 1) * T::STAGE_BYTES, ra, li.tid);
        OB::sstore(sB0 + (cur ^ 1) * T::STAGE_BYTES, rb, li.tid);
#pragma unroll
        for (int i = 0; i < T::TM; ++i) sca[i] = nsca[i];
#pragma unroll
        for (int j = 0; j < T::TN; ++j) scb[j] = nscb[j];
      }
      __syncthreads();
    }
  }
  if constexpr (T::DT == DT_I8) {
    // int32 sums -> fp32 once per K range (exact below 2^24; Stream-K partials and the epilogue work in fp32)
#pragma unroll
    for (int i = 0; i < T::TM; ++i)
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        const v4i s32 = __builtin_bit_cast(v4i, acc[i][j]);
        acc[i][j] = v4f{(float)s32.x, (float)s32.y, (float)s32.z, (float)s32.w};
      }
  }
}

// ------------------------------------------------------------------------------------------------
// epilogue: acc * (sa*sb) + bias -> cast -> store.  Lane holds C[m][n..n+3].
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float load_as_f32(const uint8_t* p, int type) {
  if (type == DT_F32) return *(const float*)p;
  if (type == DT_F16) return (float)(*(const _Float16*)p);
  uint32_t u = (uint32_t)(*(const uint16_t*)p) << 16;
  return __builtin_bit_cast(float, u);
}

// four fp32 values as four bytes of an 8-bit float format: clamped to its largest finite value (NaN kept), nearest even
template <int CT>
__device__ __forceinline__ int pack4_f8(float a, float b, float c, float d) {
  constexpr float lim = CT == DT_FP8 ? 448.f : 57344.f;
  float x[4] = {a, b, c, d};
#pragma unroll
  for (int j = 0; j < 4; ++j) x[j] = (x[j] != x[j]) ? x[j] : fminf(fmaxf(x[j], -lim), lim);
  int w;
  if constexpr (CT == DT_FP8) {
    w = __builtin_amdgcn_cvt_pk_fp8_f32(x[0], x[1], 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(x[2], x[3], w, true);
  } else {
    w = __builtin_amdgcn_cvt_pk_bf8_f32(x[0], x[1], 0, false);
    w = __builtin_amdgcn_cvt_pk_bf8_f32(x[2], x[3], w, true);
  }
  return w;
}

template <int CT>
__device__ __forceinline__ void store4(uint8_t* C, int64_t off_el, int64_t sn, v4f v, int nvalid, bool vec) {
  if constexpr (is_f8(CT)) {
    // fp32 -> e4m3fn / e5m2: clamp to the largest finite value, then round to nearest even
    // (the reference's a8w8 oracle, tests/test_matmul_a8w8_lt.py:11-38).  torch.clamp keeps NaN, and so
    // does this: fmaxf / fminf return their other argument for a NaN, which would turn a poisoned or
    // overflowed-to-NaN result into a plausible largest value.
    const int w = pack4_f8<CT>(v[0], v[1], v[2], v[3]);
    uint8_t* cp = C + off_el;
    if (vec && nvalid >= 4) { *(uint32_t*)cp = (uint32_t)w; return; }
#pragma unroll
    for (int j = 0; j < 4; ++j) if (j < nvalid) cp[j * sn] = (uint8_t)((uint32_t)w >> (8 * j));
  } else if constexpr (CT == DT_I8) {
    // fp32 -> int8: toward zero, saturated to [-128, 127] (NaN -> 0)
    uint32_t b[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float t = __builtin_truncf(v[j]);
      t = t != t ? 0.f : fminf(fmaxf(t, -128.f), 127.f);
      b[j] = (uint32_t)(int)t & 0xFFu;
    }
    uint8_t* cp = C + off_el;
    if (vec && nvalid >= 4) { *(uint32_t*)cp = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24); return; }
#pragma unroll
    for (int j = 0; j < 4; ++j) if (j < nvalid) cp[j * sn] = (uint8_t)b[j];
  } else if constexpr (CT == DT_F32) {
    float* cp = (float*)C + off_el;
    if (vec && nvalid >= 4) { *(v4f*)cp = v; return; }
#pragma unroll
    for (int j = 0; j < 4; ++j) if (j < nvalid) cp[j * sn] = v[j];
  } else {
    uint16_t h[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (CT == DT_F16) h[j] = __builtin_bit_cast(uint16_t, (_Float16)v[j]);
      else h[j] = __builtin_bit_cast(uint16_t, (__bf16)v[j]);
    }
    uint16_t* cp = (uint16_t*)C + off_el;
    if (vec && nvalid >= 4) {
      uint2 pk = {(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
      *(uint2*)cp = pk;
      return;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) if (j < nvalid) cp[j * sn] = h[j];
  }
}

template <class T, int CT>
__device__ __forceinline__ void epilogue_t(const GemmParams& p, const TileCtx& tc, v4f (&acc)[T::TM][T::TN],
                                           const LaneInfo& li) {
  float sav[T::TM];
#pragma unroll
  for (int i = 0; i < T::TM; ++i) {
    int m = tc.m0 + li.wm0 + i * 16 + li.r;
    sav[i] = (p.sa && m < tc.m_lim) ? p.sa[m] : 1.f;
  }
#pragma unroll
  for (int j = 0; j < T::TN; ++j) {
    int n = tc.n0 + li.wn0 + j * 16 + 4 * li.g;
    int nvalid = tc.n_lim - n;
    v4f sbv = {1.f, 1.f, 1.f, 1.f}, bv = {0.f, 0.f, 0.f, 0.f};
    if (tc.sb) {
#pragma unroll
      for (int q = 0; q < 4; ++q) if (q < nvalid) sbv[q] = tc.sb[n + q];
    }
    if (p.bias) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (q < nvalid) bv[q] = load_as_f32(p.bias + (int64_t)(n + q) * p.bias_stride * (p.bias_type == DT_F32 ? 4 : 2), p.bias_type);
    }
#pragma unroll
    for (int i = 0; i < T::TM; ++i) {
      int m = tc.m0 + li.wm0 + i * 16 + li.r;
      if (m >= tc.m_lim || nvalid <= 0) continue;
      v4f v = acc[i][j];
      if (p.sa) {
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = v[q] * (sav[i] * sbv[q]);
      }
      if (p.bias) {
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = v[q] + bv[q];
      }
      store4<CT>(p.C, (int64_t)m * p.c_sm + (int64_t)n * p.c_sn, p.c_sn, v, nvalid, p.c_vec);
    }
  }
}

// Full-line variant for a row-major C with 16-byte aligned rows: every wave transposes its own
// accumulator tile through a private LDS region (rows padded by 16 bytes so that the 8-byte writes
// of the 16 rows x 4 lane groups spread over the banks), then writes 16 bytes per lane, 8 lanes per
// 128-byte row segment.  No barrier is involved: a wave only reads what it wrote itself.
template <class T, int CT>
__device__ __forceinline__ void epilogue_lines(const GemmParams& p, const TileCtx& tc, v4f (&acc)[T::TM][T::TN],
                                               const LaneInfo& li, uint8_t* lds) {
  constexpr int CS = (CT == DT_F32) ? 4 : 2;
  constexpr int ROWB = T::WTN * CS;            // bytes of one wave-tile row
  constexpr int RS = ROWB + 16;                // padded LDS row stride
  constexpr int WAVES = T::WM * T::WN;
  constexpr int MAXROWS = (T::LDS_BYTES / WAVES / RS) / 16 * 16;
  constexpr int PASS_TM = (MAXROWS / 16 >= T::TM) ? T::TM : MAXROWS / 16;   // row blocks per pass
  static_assert(PASS_TM >= 1, "LDS too small for the store staging");
  static_assert(WAVES * PASS_TM * 16 * RS <= T::LDS_ALLOC - 16, "store staging must leave the broadcast word alone");
  constexpr int CPRW = ROWB / 16;              // 16-byte chunks per row
  constexpr int ROWS_PER_INST = 64 / CPRW;
  uint8_t* stage = lds + (li.tid >> 6) * (PASS_TM * 16 * RS);

  float sav[T::TM];
#pragma unroll
  for (int i = 0; i < T::TM; ++i) {
    int m = tc.m0 + li.wm0 + i * 16 + li.r;
    sav[i] = (p.sa && m < tc.m_lim) ? p.sa[m] : 1.f;
  }
  v4f sbv[T::TN], bv[T::TN];
#pragma unroll
  for (int j = 0; j < T::TN; ++j) {
    int n = tc.n0 + li.wn0 + j * 16 + 4 * li.g;
    int nvalid = tc.n_lim - n;
    sbv[j] = v4f{1.f, 1.f, 1.f, 1.f};
    bv[j] = v4f{0.f, 0.f, 0.f, 0.f};
    if (tc.sb) {
#pragma unroll
      for (int q = 0; q < 4; ++q) if (q < nvalid) sbv[j][q] = tc.sb[n + q];
    }
    if (p.bias) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (q < nvalid) bv[j][q] = load_as_f32(p.bias + (int64_t)(n + q) * p.bias_stride * (p.bias_type == DT_F32 ? 4 : 2), p.bias_type);
    }
  }
#pragma unroll
  for (int i0 = 0; i0 < T::TM; i0 += PASS_TM) {
#pragma unroll
    for (int ii = 0; ii < PASS_TM; ++ii) {
      const int i = i0 + ii;
      if (i >= T::TM) continue;
#pragma unroll
      for (int j = 0; j < T::TN; ++j) {
        v4f v = acc[i][j];
        if (p.sa) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = v[q] * (sav[i] * sbv[j][q]);
        }
        if (p.bias) {
#pragma unroll
          for (int q = 0; q < 4; ++q) v[q] = v[q] + bv[j][q];
        }
        uint8_t* dst = stage + (ii * 16 + li.r) * RS + (j * 16 + 4 * li.g) * CS;
        if constexpr (CT == DT_F32) {
          *(v4f*)dst = v;
        } else {
          uint16_t h[4];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            if constexpr (CT == DT_F16) h[q] = __builtin_bit_cast(uint16_t, (_Float16)v[q]);
            else h[q] = __builtin_bit_cast(uint16_t, (__bf16)v[q]);
          }
          uint2 pk = {(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
          *(uint2*)dst = pk;
        }
      }
    }
    // read back row-contiguous and store full lines
    constexpr int PROWS = PASS_TM * 16;
#pragma unroll
    for (int rb = 0; rb < PROWS; rb += ROWS_PER_INST) {
      const int row = rb + li.lane / CPRW;
      const int ch = li.lane % CPRW;
      const int m = tc.m0 + li.wm0 + i0 * 16 + row;
      const int n = tc.n0 + li.wn0 + ch * (16 / CS);
      if (i0 * 16 + row >= T::WTM || m >= tc.m_lim || n >= tc.n_lim) continue;
      const v4i val = *(const v4i*)(stage + row * RS + ch * 16);
      uint8_t* gp = p.C + ((int64_t)m * p.c_sm + n) * CS;
      if (n + 16 / CS <= tc.n_lim) {
        if (p.c_nt) __builtin_nontemporal_store(val, (v4i*)gp);
        else *(v4i*)gp = val;
      } else {
        const uint32_t w[4] = {(uint32_t)val.x, (uint32_t)val.y, (uint32_t)val.z, (uint32_t)val.w};
#pragma unroll
        for (int e = 0; e < 16 / CS; ++e) {
          if (n + e < tc.n_lim) {
            if constexpr (CS == 4) ((uint32_t*)gp)[e] = w[e];
            else ((uint16_t*)gp)[e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
          }
        }
      }
    }
  }
}

template <class T>
__device__ __forceinline__ void epilogue(const GemmParams& p, const TileCtx& tc, v4f (&acc)[T::TM][T::TN],
                                         const LaneInfo& li, uint8_t* lds) {
  if (p.c_line) {
    if (p.c_type == DT_BF16) epilogue_lines<T, DT_BF16>(p, tc, acc, li, lds);
    else if (p.c_type == DT_F16) epilogue_lines<T, DT_F16>(p, tc, acc, li, lds);
    else epilogue_lines<T, DT_F32>(p, tc, acc, li, lds);
    return;
  }
  if constexpr (T::DT == DT_I8) {
    if (p.c_type == DT_I8) { epilogue_t<T, DT_I8>(p, tc, acc, li); return; }
  }
  if constexpr (is_f8(T::DT)) {
    if (p.c_type == DT_FP8) { epilogue_t<T, DT_FP8>(p, tc, acc, li); return; }
    if (p.c_type == DT_E5M2) { epilogue_t<T, DT_E5M2>(p, tc, acc, li); return; }
  }
  if (p.c_type == DT_BF16) epilogue_t<T, DT_BF16>(p, tc, acc, li);
  else if (p.c_type == DT_F16) epilogue_t<T, DT_F16>(p, tc, acc, li);
  else epilogue_t<T, DT_F32>(p, tc, acc, li);
}

// ------------------------------------------------------------------------------------------------
// Stream-K partial tiles: fragment-ordered fp32 in P[slot], one float4 per lane per MFMA tile.
//
// Publisher and owner usually sit on different XCDs, whose L2s are not coherent with each other for
// ordinary accesses.  An acquire at device scope makes them so by invalidating the XCD's whole L2,
// which throws away the operand lines every other workgroup of that XCD is working from -- and a
// polling loop would do that on every poll.  So the partials and the flags move with device-scope
// accesses (sc1, as relaxed device-scope atomics use): the stores write through, the loads bypass
// stale lines and need no invalidate.  The publisher orders its stores before its flag with one release fence (the
// reference: .wt stores, .cv loads, an atomic exchange as the release, streamk_gemm.py:196-262).
// ------------------------------------------------------------------------------------------------
// Both loops are assembly with a moving scalar base and one fixed 32-bit lane offset: 32 precomputed
// 64-bit addresses next to 128 live accumulators would spill, and every reload of a spilled address
// waits for all earlier write-through stores (vmcnt is shared), which serialises them.  The s_nop in
// front of each access is required: the compiler may hand the base over in scalar registers it has
// just written with a vector instruction (v_readlane from a spill slot), the hardware wants five wait
// states between such a write and a vector-memory instruction that reads the register, and the
// compiler's hazard pass does not look inside assembly statements.
template <class T>
__device__ __forceinline__ void partial_store(float* slot, v4f (&acc)[T::TM][T::TN], int tid) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t off = (uint32_t)tid * 16u;
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j) {
      const float* base = slot + (size_t)(i * T::TN + j) * T::THREADS * 4;   // the scalar base moves, the lane offset stays
      asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 sc1" : : "v"(off), "v"(acc[i][j]), "s"(base) : "memory");
    }
#endif
}

template <class T>
__device__ __forceinline__ void partial_add(const float* slot, v4f (&acc)[T::TM][T::TN], int tid) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int NT = T::TM * T::TN;
  constexpr int BATCH = (NT % 4 == 0) ? 4 : 1;
  const uint32_t off = (uint32_t)tid * 16u;
#pragma unroll
  for (int t0 = 0; t0 < NT; t0 += BATCH) {
    v4f v[BATCH];
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      const float* base = slot + (size_t)(t0 + b) * T::THREADS * 4;
      asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2 sc1" : "=v"(v[b]) : "v"(off), "s"(base) : "memory");
    }
    // the compiler does not know that these registers are written asynchronously
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
      asm volatile("" : "+v"(v[b]));
      acc[(t0 + b) / T::TN][(t0 + b) % T::TN] += v[b];
    }
  }
#endif
}

// A value every lane holds alike, as a scalar register (an "s" operand of an assembly statement must
// be one; the compiler does not move a value it keeps in a vector register there by itself).
__device__ __forceinline__ int uniform(int x) { return __builtin_amdgcn_readfirstlane(x); }
__device__ __forceinline__ uint32_t uniform(uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); }
__device__ __forceinline__ const uint8_t* uniform(const uint8_t* p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
  return (const uint8_t*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ const float* uniform(const float* p) { return (const float*)uniform((const uint8_t*)p); }

// ------------------------------------------------------------------------------------------------
// work items: which (tile, k range) a workgroup runs next, for each schedule
// ------------------------------------------------------------------------------------------------
enum : int { WK_FULL = 0, WK_SK_PUBLISH = 1, WK_SK_OWNER = 2 };

struct Work {
  TileCtx tc;
  int it0, it1, kind;
  int64_t seg_begin, tile_first;  // Stream-K owner: global iteration where its segment / its tile begins
};

__device__ __forceinline__ void plain_tile(const GemmParams& p, int tile, int BM, int BN, TileCtx& tc) {
  int pm, pn;
  tile_coords(tile, p.tiles_m, p.tiles_n, p.group_m, p.panel_n, pm, pn);
  tc.m0 = pm * BM; tc.n0 = pn * BN; tc.m_lim = p.M; tc.n_lim = p.N;
  tc.B = p.B; tc.sb = p.sb;
}

// Grouped table: experts in order, expert e owns (its row blocks in this phase) * tiles_n tiles, m-block fastest.
// The phase this launch runs: 0 one-launch table, 1 / 2 the split tables, -1 nothing.
__device__ __forceinline__ int grouped_phase(const GemmParams& p, int grid) {
  if (p.grp_phase == 0 || !p.grp_auto) return p.grp_phase;
  int b0 = 0, b1 = 0, b2 = 0;
  for (int e = 0; e < p.num_groups; ++e) {
    const int rows = max(p.group_offsets[e + 1] - p.group_offsets[e], 0);
    const int full = rows / p.grp_big, rem = rows - full * p.grp_big;
    const bool small = rem > 0 && rem <= p.grp_thr;
    b0 += full + (rem > 0 ? 1 : 0);
    b1 += full + ((rem > 0 && !small) ? 1 : 0);
    b2 += small ? (rem + p.grp_small_bm - 1) / p.grp_small_bm : 0;
  }
  const int tn_big = p.grp_phase == 1 ? p.tiles_n : p.grp_other_tn, tn_small = p.grp_phase == 1 ? p.grp_other_tn : p.tiles_n;
  const int g_big = p.grp_phase == 1 ? grid : p.grp_other_grid, g_small = p.grp_phase == 1 ? p.grp_other_grid : grid;
  const int64_t one = 4 * (((int64_t)b0 * tn_big + g_big - 1) / g_big);
  const int64_t two = 4 * (((int64_t)b1 * tn_big + g_big - 1) / g_big) + 3 * (((int64_t)b2 * tn_small + g_small - 1) / g_small);
  const bool split = b2 > 0 && two < one;
  if (p.grp_phase == 1) return split ? 1 : 0;
  return split ? 2 : -1;
}

// the row blocks of expert e in the table of a phase: their number, the first row and the row limit
__device__ __forceinline__ int grouped_rows(const GemmParams& p, int phase, int e, int BM, int& base, int& lim) {
  const int lo = p.group_offsets[e], hi = p.group_offsets[e + 1];
  const int rows = max(hi - lo, 0);
  int mb = (rows + BM - 1) / BM;
  base = lo; lim = hi;
  if (phase != 0) {
    const int full = rows / p.grp_big, rem = rows - full * p.grp_big;
    const bool small = rem > 0 && rem <= p.grp_thr;
    if (phase == 1) { mb = full + ((rem > 0 && !small) ? 1 : 0); if (small) lim = lo + full * p.grp_big; }
    else { mb = small ? (rem + BM - 1) / BM : 0; base = lo + full * p.grp_big; }
  }
  return mb;
}

__device__ __forceinline__ bool grouped_tile(const GemmParams& p, int phase, int tile, int BM, int BN, int USZ, TileCtx& tc) {
  int acc = 0;
  for (int e = 0; e < p.num_groups; ++e) {
    int base, lim;
    const int mb = grouped_rows(p, phase, e, BM, base, lim);
    const int cnt = mb * p.tiles_n;
    if (tile < acc + cnt) {
      const int local = tile - acc;
      tc.m0 = base + (local % mb) * BM;
      tc.n0 = (local / mb) * BN;
      tc.m_lim = lim; tc.n_lim = p.N;
      tc.B = p.B + (int64_t)e * p.b_group_stride * USZ;
      tc.sb = p.sb ? p.sb + (int64_t)e * p.sb_group_stride : nullptr;
      return true;
    }
    acc += cnt;
  }
  return false;
}

__device__ __forceinline__ int grouped_total(const GemmParams& p, int phase, int BM) {
  int acc = 0;
  for (int e = 0; e < p.num_groups; ++e) {
    int base, lim;
    acc += grouped_rows(p, phase, e, BM, base, lim) * p.tiles_n;
  }
  return acc;
}

// A table of `total` tiles of `units` K units each (a unit = `unit_steps` K steps) on a resident grid of G
// workgroups: how many tiles at the table's end are cut into K ranges, one range per workgroup, instead of
// running as whole tiles.  Three plans are priced in K steps for the critical path of a workgroup: whole tiles
// only (one more round, however few tiles it holds); the tiles past the last whole round shared out; those and
// one whole round shared out (every range then covers more than a tile, so no tile has more than two pieces).
// A tile cut into n pieces costs its owner (n - 1) * fix_steps: the partial sums go through memory.
__host__ __device__ inline int sk_tail_pieces(int units, int range) {
  // the most ranges of `range` units a tile of `units` units can meet
  if (range < 1) range = 1;
  const int n = (units >= 2 ? (units - 2) / range : 0) + 2;
  return n < units ? n : units;
}
__host__ __device__ inline int sk_tail_tiles(int total, int G, int units, int unit_steps, int fix_steps) {
  if (total <= 0 || G <= 0 || units < 2) return 0;
  const int tail = total % G, rounds = total / G;
  if (tail == 0) return 0;
  long long best = (long long)(rounds + 1) * units * unit_steps;
  int pick = 0;
  for (int extra = 0; extra <= 1; ++extra) {
    if (extra > rounds) break;
    const long long skt = tail + (long long)extra * G;
    const long long all = skt * units;
    const int range = (int)(all / G);
    const long long cost = (long long)(rounds - extra) * units * unit_steps + ((all + G - 1) / G) * unit_steps +
                           (long long)(sk_tail_pieces(units, range) - 1) * fix_steps;
    if (cost < best) { best = cost; pick = (int)skt; }
  }
  return pick;
}

template <class T, bool SK>
struct Sched {
  int pid, G;
  int sk_id;              // Stream-K: position of this workgroup's iteration range = its raw workgroup id
  int next_tile;          // static / Stream-K data-parallel phase
  int step;               // work stealing: queue visit index
  int64_t start, last, q, rem;  // Stream-K iteration range of this workgroup
  int dp_tiles;
  int gphase;             // grouped: which tile table this launch runs
  int gtotal;             // grouped with a Stream-K tail: entries of that table
  bool ws_phase;          // Stream-K with work stealing: still drawing whole tiles from the queues

  __device__ __forceinline__ void init(const GemmParams& p) {
    G = gridDim.x;
    gphase = p.mode == MODE_GROUPED ? grouped_phase(p, G) : 0;
    gtotal = 0;
    pid = blockIdx.x;
    sk_id = blockIdx.x;
    if (p.mode != MODE_WS && p.num_xcds > 1) pid = chiplet_transform_chunked(pid, G, p.num_xcds, p.chunk);
    next_tile = pid;
    step = 0;
    dp_tiles = p.total_tiles - p.sk_tiles;
    start = last = q = rem = 0;
    ws_phase = false;
    if constexpr (SK) ws_phase = p.mode == MODE_SK && p.sk_ws != 0;
    if (p.mode == MODE_SK) {
      const int64_t total_sk = (int64_t)p.sk_tiles * (p.k_iters / max(1, p.sk_unit));
      q = total_sk / G; rem = total_sk % G;
      // The iteration ranges follow the order in which the hardware starts workgroups (the raw id, not
      // the XCD-remapped one): a tile is finished by the workgroup that holds its LAST iterations, so
      // every wait is for a workgroup with a lower id, which has been started already -- the exchange
      // does not need the whole grid to be resident.
      const int64_t ipt = p.k_iters / max(1, p.sk_unit);
      start = (int64_t)dp_tiles * ipt + sk_id * q + min((int64_t)sk_id, rem);
      last = (int64_t)dp_tiles * ipt + (sk_id + 1) * q + min((int64_t)sk_id + 1, rem);
    }
    if constexpr (SK) {
      if (p.mode == MODE_GROUPED && p.grp_sk && gphase >= 0) {
        // the table's real length is only known here; whole rounds first, the rest in K ranges (ordered as in MODE_SK)
        const int unit = max(1, p.sk_unit);
        const int64_t ipt = p.k_iters / unit;
        gtotal = grouped_total(p, gphase, T::BM);
        const int skt = sk_tail_tiles(gtotal, G, (int)ipt, unit, p.grp_sk_fix);
        dp_tiles = gtotal - skt;
        const int64_t total_sk = (int64_t)skt * ipt;
        q = total_sk / G; rem = total_sk % G;
        start = (int64_t)dp_tiles * ipt + sk_id * q + min((int64_t)sk_id, rem);
        last = (int64_t)dp_tiles * ipt + (sk_id + 1) * q + min((int64_t)sk_id + 1, rem);
      }
    }
    if (p.mode == MODE_WS && p.cu_mask && p.cu_mask[pid] == 0) step = 1 << 30;  // masked out: nothing to do
  }

  // The XCD x slot queues over tiles [0, total): see next().  `raw`: the workgroup id the hardware gave out (its XCD
  // and slot follow from it).
  __device__ __forceinline__ bool queue_next(const GemmParams& p, int total, int raw, Work& w, int* s_bcast, int tid) {
    const int X = p.num_xcds, S = p.counters_per_xcd;
    const int xcd = raw % X, slot = (raw / X) % S;
      if (tid < 64) {
        const int lane = tid;
        int found = -1, found_step = X * S;
        for (int base = step; base < X * S && found < 0; base += 64) {
          const int v = base + lane;
          const bool valid = v < X * S;
          const int qx = (xcd + v / S) % X;
          const int qs = (slot + v % S) % S;
          int qfirst, qcount;
          ws_queue_range(WS_QUEUES, qx * S + qs, total, X, S, 0, qfirst, qcount);
          const int bound = valid ? qcount : 0;
          int32_t* ctr = p.counters + (qx * S + qs) * COUNTER_STRIDE;
          const int seen = bound > 0 ? __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
          unsigned long long open = __ballot(bound > 0 && seen < bound);
          while (open != 0 && found < 0) {
            const int l = __builtin_ctzll(open);
            int idx = 0;
            if (lane == l) idx = atomicAdd(ctr, 1);
            idx = __shfl(idx, l);
            const int b = __shfl(bound, l), first = __shfl(qfirst, l);
            if (idx < b) { found = first + idx; found_step = base + l; }
            open &= open - 1;
          }
        }
        if (lane == 0) { s_bcast[0] = found; s_bcast[1] = found_step; }
      }
      __syncthreads();
      const int tile = s_bcast[0];
      step = s_bcast[1];
      __syncthreads();
      if (tile < 0) return false;
      plain_tile(p, tile, T::BM, T::BN, w.tc);
      return true;
  }

  // The next work item.  Every lane computes the same one, partly from values read from memory (row offsets of a
  // grouped launch, queue counters), which the compiler may keep in vector registers; what the K loops hand to
  // assembly statements as scalar operands derives from these fields, so they are made scalars here.
  __device__ __forceinline__ bool next(const GemmParams& p, Work& w, int* s_bcast, int tid) {
    const bool ok = next_item(p, w, s_bcast, tid);
    w.tc.m0 = uniform(w.tc.m0); w.tc.n0 = uniform(w.tc.n0); w.tc.m_lim = uniform(w.tc.m_lim); w.tc.n_lim = uniform(w.tc.n_lim);
    w.tc.B = uniform(w.tc.B); w.tc.sb = uniform(w.tc.sb);
    w.it0 = uniform(w.it0); w.it1 = uniform(w.it1); w.kind = uniform(w.kind);
    return ok;
  }

  __device__ __forceinline__ bool next_item(const GemmParams& p, Work& w, int* s_bcast, int tid) {
    w.it0 = 0; w.it1 = p.k_iters; w.kind = WK_FULL; w.seg_begin = w.tile_first = 0;
    if (p.mode == MODE_STATIC) {
      if (next_tile >= p.total_tiles) return false;
      plain_tile(p, next_tile, T::BM, T::BN, w.tc);
      next_tile += G;
      return true;
    }
    if (p.mode == MODE_GROUPED) {
      // the grid loops over the tile table; the first id past the table's end finishes the workgroup
      // (the host only knows an upper bound of the table's length)
      bool tail = false;
      if constexpr (SK) tail = p.grp_sk != 0;
      if (!tail) {
        if (gphase < 0 || next_tile >= p.total_tiles) return false;
        bool ok = grouped_tile(p, gphase, next_tile, T::BM, T::BN, T::USZ, w.tc);
        next_tile = ok ? next_tile + G : p.total_tiles;
        return ok;
      }
      if (gphase < 0) return false;
      if (next_tile < dp_tiles) {
        grouped_tile(p, gphase, next_tile, T::BM, T::BN, T::USZ, w.tc);
        next_tile += G;
        return true;
      }
    }
    if (p.mode == MODE_WS) {
      // Queues: one counter per (xcd, slot).  A workgroup drains its own queue, then the other
      // slots of its XCD, then the other XCDs' queues.  Visit number `step` is queue
      // ((xcd + step / S) % X, (slot + step % S) % S).  The first wave looks at 64 visits at a time:
      // every lane reads one queue's counter, the first queue (in visiting order) that still has
      // tiles gets the atomic increment, and if somebody else emptied it meanwhile the next one is
      // tried.  One round trip finds the next tile -- or finds that everything is gone -- instead of
      // one per queue.
      const int X = p.num_xcds, S = p.counters_per_xcd;
      const int xcd = pid % X, slot = (pid / X) % S;
      if (p.ws_mode != WS_QUEUES) {
        // one queue for everybody, or the XCDs' queues and the shared pool (`step` counts the queues
        // this workgroup has found empty); an XCD's counter is its slot-0 line, the pool's sits
        // behind all XCD x slot lines
        if (tid == 0) {
          int found = -1;
          if (p.ws_mode == WS_GLOBAL) {
            if (step == 0) {
              const int idx = atomicAdd(p.counters, 1);
              if (idx < p.total_tiles) found = chiplet_transform(idx, p.total_tiles, X);
              else step = 1;
            }
          } else {
            // queue order: the own XCD's queue, the shared pool, then the other XCDs' queues (those
            // only still hold tiles when their own workgroups are masked out or late)
            while (found < 0 && step <= X) {
              int line, bound, first;
              if (step == 1) { line = X * S; bound = p.ws_global; first = X * p.ws_local; }
              else { const int qx = (xcd + (step == 0 ? 0 : step - 1)) % X; line = qx * S; bound = p.ws_local; first = qx * p.ws_local; }
              int32_t* ctr = p.counters + line * COUNTER_STRIDE;
              int idx = bound;
              if (bound > 0 && __hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < bound) idx = atomicAdd(ctr, 1);
              if (idx < bound) found = first + idx;
              else ++step;
            }
          }
          s_bcast[0] = found; s_bcast[1] = step;
        }
        __syncthreads();
        const int tile = s_bcast[0];
        step = s_bcast[1];
        __syncthreads();
        if (tile < 0) return false;
        plain_tile(p, tile, T::BM, T::BN, w.tc);
        return true;
      }
      return queue_next(p, p.total_tiles, pid, w, s_bcast, tid);
    }
    if constexpr (!SK) return false;
    const bool grouped = p.mode == MODE_GROUPED;
    // MODE_SK: data-parallel tiles first (from the work-stealing queues when asked for, reference
    // kernels/streamk_gemm_work_stealing.py:9-418), then this workgroup's share of the Stream-K iterations
    if (grouped) {
      // (its whole tiles were handed out above)
    } else if (ws_phase) {
      if (queue_next(p, dp_tiles, sk_id, w, s_bcast, tid)) return true;
      ws_phase = false;
      step = 0;
    } else if (p.sk_ws == 0 && next_tile < dp_tiles) {
      plain_tile(p, next_tile, T::BM, T::BN, w.tc);
      next_tile += G;
      return true;
    }
    // The range is walked from its end: the piece that does not reach its tile's end (at most one,
    // the head of the range's last tile) comes first and is published at once; the pieces that do
    // reach a tile's end finish that tile, adding what lower workgroups published long before.
    if (start >= last) return false;
    const int unit = max(1, p.sk_unit);
    const int ipt = p.k_iters / unit;
    const int tile = (int)((last - 1) / ipt);
    const int64_t tile_first = (int64_t)tile * ipt;
    const int64_t tile_end = tile_first + ipt;
    const int64_t begin = max(tile_first, start);
    if (grouped) grouped_tile(p, gphase, tile, T::BM, T::BN, T::USZ, w.tc);
    else plain_tile(p, tile, T::BM, T::BN, w.tc);
    w.it0 = (int)(begin - tile_first) * unit;
    w.it1 = (int)(last - tile_first) * unit;
    w.kind = (last != tile_end) ? WK_SK_PUBLISH : WK_SK_OWNER;
    w.seg_begin = begin; w.tile_first = tile_first;
    last = begin;
    return true;
  }
};

// What the last workgroup of a Stream-K launch to leave does: advance the launch count the workspace keeps (every
// workgroup has read it before it gets here) and rearm the work-stealing queues if the launch drew from them.
__device__ __forceinline__ void sk_leave(const GemmParams& p, uint32_t epoch, int tid) {
  if (!(p.mode == MODE_SK || (p.mode == MODE_GROUPED && p.grp_sk)) || tid != 0 || (p.epoch != EPOCH_ON_DEVICE && !p.sk_ws)) return;
  const uint32_t done = atomicAdd(p.ctl + CTL_DONE, 1u);
  if (done != gridDim.x - 1) return;
  if (p.sk_ws)
    for (int qi = 0; qi <= p.num_xcds * p.counters_per_xcd; ++qi)
      __hip_atomic_store(p.counters + qi * COUNTER_STRIDE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (p.epoch == EPOCH_ON_DEVICE) __hip_atomic_store(p.ctl + CTL_EPOCH, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(p.ctl + CTL_DONE, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// SK = false: data-parallel, work-stealing and grouped schedules (every work item is a whole tile).
// SK = true: adds the Stream-K tail with its partial-tile publish / fixup paths.  Two kernels, so that
// the accumulator-heavy fixup code cannot push the common path into register spills.
template <class T, bool SK>
__global__ __launch_bounds__(T::THREADS, T::MINB) void gemm_kernel(const GemmParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[T::LDS_ALLOC];
  int& s_bcast = *(int*)(lds + T::LDS_ALLOC - 16);
  LaneInfo li;
  li.tid = threadIdx.x;
  li.lane = li.tid & 63;
  li.r = li.lane & 15;
  li.g = li.lane >> 4;
  const int wave = li.tid >> 6;
  li.wm0 = (wave / T::WN) * T::WTM;
  li.wn0 = (wave % T::WN) * T::WTN;
  v4f acc[T::TM][T::TN];

  Sched<T, SK> sched;
  sched.init(p);
  Work w;
  bool failed = false;   // a Stream-K wait ran into its poll bound (the status word tells the host)
  // The tag of this launch's partial tiles: the caller's epoch, or one more than the count the
  // workspace keeps itself (control word CTL_EPOCH, which the last workgroup to leave advances) --
  // the form a launch replayed from a captured graph needs, whose arguments cannot change.
  uint32_t epoch = p.epoch;
  if constexpr (SK) {
    if (p.epoch == EPOCH_ON_DEVICE) epoch = __hip_atomic_load(p.ctl + CTL_EPOCH, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
  }
  while (sched.next(p, w, &s_bcast, li.tid)) {
    __syncthreads();  // the previous item's store staging may still be read by slower waves
    mainloop<T, !SK>(p, w.tc, w.it0, w.it1, acc, lds, li);
    if constexpr (SK) {
    if (w.kind == WK_FULL) {
      // whole tiles get their own copy of the epilogue: sharing the one behind the fixup code makes
      // the compiler park the accumulators in scratch on this, the common, path too
      epilogue<T>(p, w.tc, acc, li, lds);
      continue;
    }
    if (w.kind == WK_SK_PUBLISH) {
      // not the tile's last segment: publish the partial, tagged with this launch's epoch
      partial_store<T>(p.P + (size_t)sched.sk_id * (T::BM * T::BN), acc, li.tid);
      __builtin_amdgcn_s_waitcnt(0x0070);   // this wave's write-through stores have left the CU
      __syncthreads();                      // ... and so have everybody else's
      if (li.tid == 0) {
        // one L2 write-back for the workgroup (it covers every wave's stores), then the flag
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
        __hip_atomic_store(p.flags + sched.sk_id, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      continue;
    }
    if (w.kind == WK_SK_OWNER) {
      // owner of the tile (it holds the last iterations): add the partials of the workgroups before it,
      // nearest first -- a fixed order, so the sum is the same in every launch
      int nxt = sched.sk_id - 1;
      int64_t cur_begin = w.seg_begin;
      while (cur_begin > w.tile_first) {
        if (li.tid == 0) {
          uint32_t spins = 0;
          int ok = 1;
          while (__hip_atomic_load(p.flags + nxt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != epoch) {
            if (++spins >= p.spin_limit) { ok = 0; break; }
            __builtin_amdgcn_s_sleep(2);
          }
          s_bcast = ok;
        }
        __syncthreads();
        int ok = s_bcast;
        __syncthreads();
        if (!ok) {
          // a partner did not publish within the bound (the bound is too tight, or the device is shared
          // with something that starves it): the tile cannot
          // be finished.  It is stored as NaN so that nobody mistakes stale memory for a result, and the
          // status word tells the host.  The workgroup then goes on with the rest of its work list: every
          // tile it owns ends up either finished or NaN, never untouched.
          failed = true;
          const float nanv = __builtin_nanf("");
#pragma unroll
          for (int i = 0; i < T::TM; ++i)
#pragma unroll
            for (int j = 0; j < T::TN; ++j) acc[i][j] = v4f{nanv, nanv, nanv, nanv};
          break;
        }
        partial_add<T>(p.P + (size_t)nxt * (T::BM * T::BN), acc, li.tid);
        cur_begin -= sched.q + (nxt < sched.rem ? 1 : 0);
        --nxt;
      }
    }
    }
    epilogue<T>(p, w.tc, acc, li, lds);
  }
  if constexpr (SK) {
    if (failed && li.tid == 0) atomicExch(p.ctl + CTL_STATUS, 1u);
    sk_leave(p, epoch, li.tid);
  }
  if (!SK && p.mode == MODE_WS && li.tid == 0) {
    // the last workgroup to leave rearms the queues for the next launch
    uint32_t done = atomicAdd(p.ctl + CTL_DONE, 1u);
    if (done == gridDim.x - 1) {
      for (int qi = 0; qi <= p.num_xcds * p.counters_per_xcd; ++qi)   // (the last line is the shared pool's)
        __hip_atomic_store(p.counters + qi * COUNTER_STRIDE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(p.ctl + CTL_DONE, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace tb
