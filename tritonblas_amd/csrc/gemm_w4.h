// 256x256 tile GEMM with four waves (one per SIMD), 128x128 wave tiles and a hand-scheduled K loop.
//
// The compiler-scheduled kernels of gemm_device.h run the 256x256 tile with eight waves (128x64 wave
// tiles): with one wave per SIMD every LDS wait of compiler-ordered code stalls the only wave there is,
// and 256 accumulator registers leave the allocator no room.  Here the K loop of one output tile is one
// assembly statement (gen_w4.py writes it): the accumulators live in a[0:255], fragments and scales
// in v[0:191], every MFMA, LDS read, LDS-direct copy and wait is placed by hand.  Everything around
// it -- tile schedule, per-tile addresses, epilogue -- stays C++.  The wave tile is a quarter of the
// 8-wave kernels' K-step LDS traffic less (128 KB instead of 196 KB of fragment reads per 64 KB copied).
//
// Differences from the 8-wave kernels that matter to callers: K must be a multiple of two K steps and
// there is no Stream-K variant (whole tiles only: data-parallel, work-stealing and grouped schedules).
// Sums are formed in the same order (same MFMA instruction, same K grouping, K steps in ascending
// order), so results are bit-identical to the 8-wave kernels'.
//
// Output layout.  The B tile is the first MFMA operand, so a lane holds four consecutive output
// columns of one row per MFMA tile.  The rows of the B tile are copied into LDS in a permuted order
// (LDS row 16j + 4g + e of a wave's 128 holds column 32(j/2) + 8g + 4(j%2) + e), which makes the eight
// values a lane holds for MFMA tiles 2q and 2q+1 eight consecutive columns: the epilogue stores them
// as one 16-byte write per lane straight from registers (64 contiguous bytes per row and instruction),
// with no LDS staging -- the LDS already belongs to the next tile's first K steps by then.
#pragma once
#include <utility>
#include "gemm_variants.h"

namespace tb {

typedef int v16i __attribute__((ext_vector_type(16)));

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// accumulator register a[N] (written by the K loop statement; the compiler never allocates these);
// INT: the K loop left an int32 sum there
template <int N, bool INT = false>
__device__ __forceinline__ float acc_read() {
  if constexpr (INT) {
    int x;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(N));
    return (float)x;
  } else {
    float x;
    asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(N));
    return x;
  }
}

// what the K loop needs to know about one output tile
struct W4TileArgs {
  const uint8_t* A;      // first row of the tile, k = 0
  const uint8_t* B;
  const uint8_t* mxa;    // FP4: scale rows
  const uint8_t* mxb;
  v16i off;              // byte offsets of this lane's 8 + 8 copy chunks from (A, B) at a K step's origin
  uint32_t sca, scb;     // FP4: byte offsets of this lane's scale rows from (mxa, mxb)
};

struct W4Lane {
  int r, g, wm0, wn0;
  uint32_t c16;          // swizzled chunk (byte offset) this lane copies in every row it copies
  int pa, pb;            // tile row this lane copies with copy instruction 0 (instruction i: + 32 i)
  int sra, srb;          // FP4: tile rows whose scales this lane copies
};

// it0: first K step of the work item (a Stream-K piece starts inside the tile's K range)
template <class T>
__device__ __forceinline__ void w4_tile_args(const GemmParams& p, const TileCtx& tc, int it0, const W4Lane& ln, W4TileArgs& t) {
  const int rva = tc.m_lim - tc.m0, rvb = tc.n_lim - tc.n0;
  const uint32_t sra = (uint32_t)p.a_sr * T::USZ, srb = (uint32_t)p.b_sr * T::USZ;   // row strides in bytes
  t.A = p.A + (int64_t)tc.m0 * p.a_sr * T::USZ + (int64_t)it0 * 128;
  t.B = tc.B + (int64_t)tc.n0 * p.b_sr * T::USZ + (int64_t)it0 * 128;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    t.off[i] = (int)((uint32_t)min(i * 32 + ln.pa, rva - 1) * sra + ln.c16);
    t.off[8 + i] = (int)((uint32_t)min(i * 32 + ln.pb, rvb - 1) * srb + ln.c16);
  }
  if constexpr (T::DT == DT_FP4) {
    t.mxa = p.mxa + (int64_t)tc.m0 * p.mxa_sr + it0 * 8;      // (eight E8M0 bytes per row and K step)
    t.mxb = p.mxb + (int64_t)tc.n0 * p.mxb_sr + it0 * 8;
    t.sca = (uint32_t)min(ln.sra, rva - 1) * (uint32_t)p.mxa_sr;
    t.scb = (uint32_t)min(ln.srb, rvb - 1) * (uint32_t)p.mxb_sr;
  } else {
    t.mxa = t.mxb = nullptr;
    t.sca = t.scb = 0;
  }
}

// acc * (sa*sb) + bias -> cast -> store, straight from the accumulator registers.  Lane (g, r) of wave
// (wm, wn) holds, for row block i and column group q, C[m0 + wm0 + 16i + r][n0 + wn0 + 32q + 8g + 0..7].
template <class T, int CT>
__device__ __forceinline__ void epilogue_w4(const GemmParams& p, const TileCtx& tc, const W4Lane& ln) {
  float sav[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = tc.m0 + ln.wm0 + i * 16 + ln.r;
    sav[i] = (p.sa && m < tc.m_lim) ? p.sa[m] : 1.f;
  }
  static_for<4>([&](auto Q) {
    constexpr int q = decltype(Q)::value;
    const int n = tc.n0 + ln.wn0 + 32 * q + 8 * ln.g;
    const int nvalid = tc.n_lim - n;
    float sbv[8], bv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sbv[e] = (tc.sb && e < nvalid) ? tc.sb[n + e] : 1.f;
      bv[e] = (p.bias && e < nvalid)
                  ? load_as_f32(p.bias + (int64_t)(n + e) * p.bias_stride * (p.bias_type == DT_F32 ? 4 : 2), p.bias_type)
                  : 0.f;
    }
    static_for<8>([&](auto I) {
      constexpr int i = decltype(I)::value;
      float v[8];
      static_for<8>([&](auto E) {
        constexpr int e = decltype(E)::value;
        v[e] = acc_read<((i * 8 + 2 * q + (e >> 2)) * 4 + (e & 3)), T::DT == DT_I8>();
      });
      const int m = tc.m0 + ln.wm0 + i * 16 + ln.r;
      if (m >= tc.m_lim || nvalid <= 0) return;
      if (p.sa) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = v[e] * (sav[i] * sbv[e]);
      }
      if (p.bias) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = v[e] + bv[e];
      }
      if constexpr (is_f8(CT)) {
        // fp32 -> e4m3fn / e5m2: clamp to the largest finite value (NaN stays NaN, as torch.clamp keeps it), round to
        // nearest even; eight consecutive output columns are eight bytes
        const int w0 = pack4_f8<CT>(v[0], v[1], v[2], v[3]);
        const int w1 = pack4_f8<CT>(v[4], v[5], v[6], v[7]);
        uint8_t* cp = p.C + ((int64_t)m * p.c_sm + (int64_t)n * p.c_sn);
        if (p.c_vec && p.c_sn == 1 && nvalid >= 8 && (((uintptr_t)cp) & 7) == 0) {
          *(uint2*)cp = uint2{(uint32_t)w0, (uint32_t)w1};
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e < nvalid) cp[e * p.c_sn] = (uint8_t)((uint32_t)(e < 4 ? w0 : w1) >> (8 * (e & 3)));
        }
      } else if constexpr (CT == DT_F32) {
        float* cp = (float*)p.C + ((int64_t)m * p.c_sm + (int64_t)n * p.c_sn);
        if (p.c_line && nvalid >= 8) {
          const v4f lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
          if (p.c_nt) { __builtin_nontemporal_store(lo, (v4f*)cp); __builtin_nontemporal_store(hi, (v4f*)cp + 1); }
          else { *(v4f*)cp = lo; *((v4f*)cp + 1) = hi; }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) if (e < nvalid) cp[e * p.c_sn] = v[e];
        }
      } else {
        uint32_t h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if constexpr (CT == DT_F16) h[e] = __builtin_bit_cast(uint16_t, (_Float16)v[e]);
          else h[e] = __builtin_bit_cast(uint16_t, (__bf16)v[e]);
        }
        uint16_t* cp = (uint16_t*)p.C + ((int64_t)m * p.c_sm + (int64_t)n * p.c_sn);
        if (p.c_line && nvalid >= 8) {
          const v4i pk = {(int)(h[0] | (h[1] << 16)), (int)(h[2] | (h[3] << 16)), (int)(h[4] | (h[5] << 16)), (int)(h[6] | (h[7] << 16))};
          if (p.c_nt) __builtin_nontemporal_store(pk, (v4i*)cp);
          else *(v4i*)cp = pk;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) if (e < nvalid) cp[e * p.c_sn] = (uint16_t)h[e];
        }
      }
    });
  });
}

// Fast path of the epilogue: the whole 256x256 tile lies inside C, C rows are 16-byte aligned with
// unit column stride, 16-bit output, no bias, scale vectors 16-byte aligned.  No per-element bounds
// handling, and exactly 32 stores per wave, issued as assembly so that the count is known: the next
// tile's K loop waits for its first copies with "at most N younger memory operations in flight" and
// has to know how many of those are this epilogue's stores.
template <class T, int CT, bool NT>
__device__ __forceinline__ void epilogue_w4_fast(const GemmParams& p, const TileCtx& tc, const W4Lane& ln) {
  const int mrow = tc.m0 + ln.wm0 + ln.r;
  const int ncol = tc.n0 + ln.wn0 + 8 * ln.g;
  float sav[8];
  v4f sbv[8];
  if (p.sa) {
#pragma unroll
    for (int i = 0; i < 8; ++i) sav[i] = p.sa[mrow + i * 16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      sbv[2 * q] = *(const v4f*)(tc.sb + ncol + 32 * q);
      sbv[2 * q + 1] = *(const v4f*)(tc.sb + ncol + 32 * q + 4);
    }
  }
  uint16_t* c0 = (uint16_t*)p.C + ((int64_t)mrow * p.c_sm + ncol);
  static_for<8>([&](auto I) {
    constexpr int i = decltype(I)::value;
    uint16_t* crow = c0 + (int64_t)(i * 16) * p.c_sm;
    static_for<4>([&](auto Q) {
      constexpr int q = decltype(Q)::value;
      float v[8];
      static_for<8>([&](auto E) {
        constexpr int e = decltype(E)::value;
        v[e] = acc_read<((i * 8 + 2 * q + (e >> 2)) * 4 + (e & 3)), T::DT == DT_I8>();
      });
      if (p.sa) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = v[e] * (sav[i] * sbv[2 * q + (e >> 2)][e & 3]);
      }
      uint32_t h[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if constexpr (CT == DT_F16) h[e] = __builtin_bit_cast(uint16_t, (_Float16)v[e]);
        else h[e] = __builtin_bit_cast(uint16_t, (__bf16)v[e]);
      }
      const v4i pk = {(int)(h[0] | (h[1] << 16)), (int)(h[2] | (h[3] << 16)), (int)(h[4] | (h[5] << 16)), (int)(h[6] | (h[7] << 16))};
      uint16_t* const dst = crow;   // (assembly operands do not capture: name a local of this lambda)
#ifdef W4_LAB_NOSTORE
      if (p.debug == 12345)         // measurement build: no stores (the condition keeps the code alive)
#endif
      // (the s_nop: a store of more than 8 bytes reads its data registers a little after it issues, and the
      // compiler, which inserts the wait states for its own stores, cannot see into this statement -- without
      // them the int8 kernel's next conversion overwrote the first data register for some lanes)
      if constexpr (NT) asm volatile("global_store_dwordx4 %0, %1, off offset:%2 nt\n\ts_nop 1" : : "v"(dst), "v"(pk), "n"(q * 64) : "memory");
      else asm volatile("global_store_dwordx4 %0, %1, off offset:%2\n\ts_nop 1" : : "v"(dst), "v"(pk), "n"(q * 64) : "memory");
    });
  });
}

// ---- Stream-K pieces ---------------------------------------------------------------------------------------
// A partial tile travels in the order the accumulators have it: MFMA tile t = 8 i + j of wave w is one 16-byte
// value per lane at float offset ((w * 64 + t) * 64 + lane) * 4 of the workgroup's slot -- 1 KB per store, no
// layout change on either side.  Device-scope (sc1) accesses: publisher and owner usually sit on different XCDs.
template <class T>
__device__ __forceinline__ void partial_store_w4(float* slot, int wave, int lane) {
  const uint32_t off = (uint32_t)lane * 16u;
  static_for<64>([&](auto TT) {
    constexpr int t = decltype(TT)::value;
    v4f v;
    v[0] = acc_read<t * 4 + 0, T::DT == DT_I8>(); v[1] = acc_read<t * 4 + 1, T::DT == DT_I8>();
    v[2] = acc_read<t * 4 + 2, T::DT == DT_I8>(); v[3] = acc_read<t * 4 + 3, T::DT == DT_I8>();
    const float* base = slot + (size_t)(wave * 64 + t) * 256;
    const uint32_t o = off;   // (assembly operands do not capture: name locals of this lambda)
    // (the wait states behind the store: it still reads its data registers for a moment after it issues, and the
    // compiler, which cannot see into the statement, lets the next accumulator read reuse them at once)
    asm volatile("s_nop 4\n\tglobal_store_dwordx4 %0, %1, %2 sc1\n\ts_nop 1" : : "v"(o), "v"(v), "s"(base) : "memory");
  });
}

// The tile's owner: its own sums plus the partial tiles of workgroups id_hi, id_hi - 1, ... (n of them, nearest
// first: a fixed order), then acc * (sa*sb) + bias -> cast -> store with bounds.  poison: a partner did not
// publish in time, the tile is stored as NaN.
template <class T, int CT>
__device__ __forceinline__ void epilogue_w4_owner(const GemmParams& p, const TileCtx& tc, const W4Lane& ln, int wave, int lane,
                                                  int id_hi, int n, bool poison) {
  const uint32_t off = (uint32_t)lane * 16u;
  float sav[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = tc.m0 + ln.wm0 + i * 16 + ln.r;
    sav[i] = (p.sa && m < tc.m_lim) ? p.sa[m] : 1.f;
  }
  static_for<4>([&](auto Q) {
    constexpr int q = decltype(Q)::value;
    // the 16 MFMA tiles (i, 2q) and (i, 2q + 1), i = 0..7, of this column group
    v4f v[16];
    static_for<16>([&](auto X) {
      constexpr int x = decltype(X)::value;
      constexpr int t = (x >> 1) * 8 + 2 * q + (x & 1);
      v[x][0] = acc_read<t * 4 + 0, T::DT == DT_I8>(); v[x][1] = acc_read<t * 4 + 1, T::DT == DT_I8>();
      v[x][2] = acc_read<t * 4 + 2, T::DT == DT_I8>(); v[x][3] = acc_read<t * 4 + 3, T::DT == DT_I8>();
    });
    const uint32_t o = off;   // (assembly operands do not capture: name locals of this lambda)
    for (int k = 0; k < n; ++k) {
      const float* slot = p.P + (size_t)(id_hi - k) * (256 * 256);
      v4f part[16];
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const int t = (x >> 1) * 8 + 2 * q + (x & 1);
        const float* base = slot + (size_t)(wave * 64 + t) * 256;
        asm volatile("s_nop 4\n\tglobal_load_dwordx4 %0, %1, %2 sc1" : "=v"(part[x]) : "v"(o), "s"(base) : "memory");
      }
      // (the compiler does not know that these registers are written asynchronously)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        asm volatile("" : "+v"(part[x]));
        v[x] += part[x];
      }
    }
    const int ncol = tc.n0 + ln.wn0 + 32 * q + 8 * ln.g;
    const int nvalid = tc.n_lim - ncol;
    float sbv[8], bv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sbv[e] = (tc.sb && e < nvalid) ? tc.sb[ncol + e] : 1.f;
      bv[e] = (p.bias && e < nvalid)
                  ? load_as_f32(p.bias + (int64_t)(ncol + e) * p.bias_stride * (p.bias_type == DT_F32 ? 4 : 2), p.bias_type)
                  : 0.f;
    }
    static_for<8>([&](auto I) {
      constexpr int i = decltype(I)::value;
      const int m = tc.m0 + ln.wm0 + i * 16 + ln.r;
      if (m >= tc.m_lim || nvalid <= 0) return;
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float x = v[2 * i + (e >> 2)][e & 3];
        if (p.sa) x = x * (sav[i] * sbv[e]);
        if (p.bias) x = x + bv[e];
        o[e] = poison ? __builtin_nanf("") : x;
      }
      if constexpr (CT == DT_F32) {
        float* cp = (float*)p.C + ((int64_t)m * p.c_sm + (int64_t)ncol * p.c_sn);
#pragma unroll
        for (int e = 0; e < 8; ++e) if (e < nvalid) cp[e * p.c_sn] = o[e];
      } else {
        uint16_t* cp = (uint16_t*)p.C + ((int64_t)m * p.c_sm + (int64_t)ncol * p.c_sn);
        uint32_t h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if constexpr (CT == DT_F16) h[e] = __builtin_bit_cast(uint16_t, (_Float16)o[e]);
          else h[e] = __builtin_bit_cast(uint16_t, (__bf16)o[e]);
        }
        if (p.c_line && nvalid >= 8) {
          const v4i pk = {(int)(h[0] | (h[1] << 16)), (int)(h[2] | (h[3] << 16)), (int)(h[4] | (h[5] << 16)), (int)(h[6] | (h[7] << 16))};
          *(v4i*)cp = pk;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) if (e < nvalid) cp[e * p.c_sn] = (uint16_t)h[e];
        }
      }
    });
  });
}

// operands every kind of K loop statement takes
#define W4_COMMON_OPERANDS                                                                                              \
  [offc] "{v[192:207]}"(cur.off), [offn] "{v[208:223]}"(nxt.off), [fa] "{v[224:231]}"(fa), [A] "s"(sA), [B] "s"(sB),     \
      [An] "s"(sAn), [Bn] "s"(sBn), [wl] "s"(wl), [kh] "s"(s_kh), [first] "s"(s_first), [nst] "s"(s_nst), [fe] "s"(s_fe), \
      [cprev] "s"(s_cprev), [cstep] "s"(s_cstep)

#ifdef W4_LAB_TS
// measurement build: when (constant 100 MHz counter) every workgroup started and finished each of its tiles (one array per
// translation unit that includes this file; the one the host reads back is that of the 8-bit float kernels)
static __device__ unsigned long long w4_lab_ts[1024 * 32];
#endif

// SK: the schedule may end in a Stream-K tail (pieces of a tile's K range, cut at multiples of four K steps:
// GemmParams::sk_unit = 4), with the partial-tile exchange of gemm_kernel<T, true>.
template <class T, bool SK = false>
__global__ __launch_bounds__(256, 1) void gemm_kernel_w4(const GemmParams p) {
  static_assert(T::BM == 256 && T::BN == 256 && T::BKB == 128 && T::WM == 2 && T::WN == 2 && T::STAGES == 2, "fixed shape");
  static_assert(is_f8(T::DT) || T::DT == DT_FP4 || T::DT == DT_BF16 || T::DT == DT_F16 || T::DT == DT_I8, "element types with a generated K loop");
  // two stages, the FP4 scale buffers (16 KB), 1 KB per wave for epilogue scales, the schedule's broadcast word
  __shared__ __attribute__((aligned(16))) uint8_t lds[W4_LDS_BYTES];
  int& s_bcast = *(int*)(lds + W4_LDS_BYTES - 16);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) uint8_t*)lds);

  W4Lane ln;
  ln.r = lane & 15;
  ln.g = lane >> 4;
  ln.wm0 = (wave >> 1) * 128;
  ln.wn0 = (wave & 1) * 128;
  const int l8 = lane >> 3;
  // copy instruction i of this wave fills LDS rows 32i + 8*wave + l8 (A rows, then B rows), chunk slot
  // lane % 8; the row's swizzle mask is (row % 8) ^ ((row / 8) & 1) = l8 ^ (wave & 1)
  ln.c16 = (uint32_t)(((lane & 7) ^ l8 ^ (wave & 1)) << 4);
  ln.pa = wave * 8 + l8;
  // B: LDS row rho = 16j + 4g' + e (within a wave's 128 rows) takes tile row 32(j/2) + 8g' + 4(j%2) + e
  ln.pb = ((wave & 1) * 2 + (l8 >> 2)) * 8 + (wave >> 1) * 4 + (l8 & 3);
  ln.sra = wave * 64 + lane;
  {
    const int rho = ln.sra & 127, j = rho >> 4, gg = (rho >> 2) & 3, e = rho & 3;
    ln.srb = (ln.sra & 128) + (j >> 1) * 32 + gg * 8 + (j & 1) * 4 + e;
  }
  // fragment read addresses: lane (g, r) reads chunks 2g and 2g+1 of row (wave row base + 16t + r)
  v8i fa;
  {
    const int m = (ln.r & 7) ^ (ln.r >> 3);
    const uint32_t lo = (uint32_t)(((2 * ln.g) ^ m) << 4);
    const uint32_t a0 = lds0 + (uint32_t)(ln.wm0 + ln.r) * 128u + lo;
    const uint32_t b0 = lds0 + 32768u + (uint32_t)(ln.wn0 + ln.r) * 128u + lo;
    fa[0] = (int)a0; fa[1] = (int)(a0 ^ 16u); fa[2] = (int)b0; fa[3] = (int)(b0 ^ 16u);
    fa[4] = (int)(a0 + 65536u); fa[5] = (int)((a0 ^ 16u) + 65536u); fa[6] = (int)(b0 + 65536u); fa[7] = (int)((b0 ^ 16u) + 65536u);
  }
  const uint32_t wl = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + (uint32_t)wave * 1024u));

  Sched<T, SK> sched;
  sched.init(p);
  uint32_t epoch = p.epoch;
  bool failed = false;
  if constexpr (SK) {
    if (p.epoch == EPOCH_ON_DEVICE) epoch = __hip_atomic_load(p.ctl + CTL_EPOCH, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
  }
#ifdef W4_LAB_XCD_DELAY
  // measurement build: the workgroups of the odd XCDs start (debug >> 8) * 8128 cycles late, so that the XCDs
  // reach their tile changes (and the store bursts of the fused epilogues) at different times
  if (blockIdx.x & 1)
    for (int i = 0; i < (p.debug >> 8); ++i) __builtin_amdgcn_s_sleep(127);
#endif
#ifdef W4_LAB_TS
  int ts_n = 0;
  if (tid == 0 && blockIdx.x < 1024) w4_lab_ts[blockIdx.x * 32 + ts_n] = __builtin_amdgcn_s_memrealtime();
  ++ts_n;
#endif
  Work w, wnext;
  bool have = sched.next(p, w, &s_bcast, tid);
  int first = 1;
  int nst = 0;             // 1: the previous tile's epilogue issued exactly 32 stores per wave (its fast path)
  uint32_t scbuf = 0;
  // Fused epilogue: a full tile with bf16 output (and, for FP8, both scale vectors; for the other
  // kinds, none) is not stored by the code below but by the NEXT tile's K loop, which reads each
  // accumulator row block out just before its first K step overwrites it.  The last tile of a workgroup
  // always takes the code below.  An FP8 K loop copies its own tile's scale vectors into LDS for that.
  int fe = 0;                       // 1: the previous tile's sums are still in the accumulators
  const uint8_t* cprev = (const uint8_t*)p.C;   // C[first row of the wave's quarter][its first column] of that tile
  const bool fe_shape = p.c_line && !p.bias && (p.c_type == DT_BF16 || p.c_type == DT_F16) && p.c_sm < (1 << 26) && (p.debug & 4) == 0 &&
                        ((is_f8(T::DT) || T::DT == DT_I8) == (p.sa != nullptr));
  // a lane's C offset from cprev, the same in every row block (rows of a row block are c_sm apart);
  // lane * 4; where the lane finds the scales of its rows 16 i + r and of its columns 32 q + 8 g + 0..7
  v4i eo;
  eo[0] = (int)(((uint32_t)ln.r * (uint32_t)p.c_sm + 8u * (uint32_t)ln.g) * 2u);
  eo[1] = lane * 4;
  eo[2] = (int)(lds0 + (uint32_t)W4_EPS_OFFSET + (uint32_t)wave * 1024u + (uint32_t)ln.r * 4u);
  eo[3] = (int)(lds0 + (uint32_t)W4_EPS_OFFSET + (uint32_t)wave * 1024u + 512u + (uint32_t)ln.g * 32u);
  const uint32_t s_cstep = uniform((uint32_t)p.c_sm * 32u);
  while (have) {
    // the tile after this one: its first two K steps are requested during this tile's last two.  With
    // none left the copies read this tile's first steps again; nobody uses them.
    const bool have_next = sched.next(p, wnext, &s_bcast, tid);
    if (!have_next) wnext = w;
    W4TileArgs cur, nxt;
    w4_tile_args<T>(p, w.tc, w.it0, ln, cur);
    w4_tile_args<T>(p, wnext.tc, wnext.it0, ln, nxt);
    const int kh = (w.it1 - w.it0) >> 1;
    const bool fast = p.c_line && !p.bias && p.c_type != DT_F32 && w.tc.m0 + 256 <= w.tc.m_lim && w.tc.n0 + 256 <= w.tc.n_lim &&
                      (!p.sa || (((uintptr_t)w.tc.sb & 15) == 0));
    const bool regs = (is_f8(T::DT) || T::DT == DT_I8) && fast && p.sa;    // the K loop copies this tile's scale vectors
    const uint8_t *sA = uniform(cur.A), *sB = uniform(cur.B), *sAn = uniform(nxt.A), *sBn = uniform(nxt.B);
    const int s_kh = uniform(kh), s_first = uniform(first), s_nst = uniform(nst), s_fe = uniform(fe);
    const uint8_t* s_cprev = uniform(cprev);
    scbuf = uniform(scbuf);
#ifdef W4_LAB_TS2
    // (with -DW4_LAB_TS -DW4_LAB_TS2: two stamps per tile, in front of and behind its K loop statement, instead of one)
    if (tid == 0 && blockIdx.x < 1024 && ts_n < 31) w4_lab_ts[blockIdx.x * 32 + ts_n] = __builtin_amdgcn_s_memrealtime();
    ++ts_n;
#endif
    if constexpr (is_f8(T::DT) || T::DT == DT_I8) {
      // (a tile without scales or off the fast path loads 512 bytes of its operands instead; nobody uses them)
      const uint8_t* s_sap = uniform(regs ? (const uint8_t*)(p.sa + w.tc.m0 + ln.wm0) : cur.A);
      const uint8_t* s_sbp = uniform(regs ? (const uint8_t*)(w.tc.sb + w.tc.n0 + ln.wn0) : cur.B);
      if constexpr (T::DT == DT_FP8) {
        asm volatile(
#include "w4_kloop_fp8.inc"
            : [scbuf] "+s"(scbuf)
            : W4_COMMON_OPERANDS, [eo] "{v[240:243]}"(eo), [sap] "s"(s_sap), [sbp] "s"(s_sbp)
            :
#include "w4_clobbers_fp8.inc"
        );
      } else if constexpr (T::DT == DT_E5M2) {
        asm volatile(
#include "w4_kloop_e5m2.inc"
            : [scbuf] "+s"(scbuf)
            : W4_COMMON_OPERANDS, [eo] "{v[240:243]}"(eo), [sap] "s"(s_sap), [sbp] "s"(s_sbp)
            :
#include "w4_clobbers_e5m2.inc"
        );
      } else if constexpr (T::DT == DT_E4E5) {
        asm volatile(
#include "w4_kloop_e4e5.inc"
            : [scbuf] "+s"(scbuf)
            : W4_COMMON_OPERANDS, [eo] "{v[240:243]}"(eo), [sap] "s"(s_sap), [sbp] "s"(s_sbp)
            :
#include "w4_clobbers_e4e5.inc"
        );
      } else if constexpr (T::DT == DT_E5E4) {
        asm volatile(
#include "w4_kloop_e5e4.inc"
            : [scbuf] "+s"(scbuf)
            : W4_COMMON_OPERANDS, [eo] "{v[240:243]}"(eo), [sap] "s"(s_sap), [sbp] "s"(s_sbp)
            :
#include "w4_clobbers_e5e4.inc"
        );
      } else {
        asm volatile(
#include "w4_kloop_i8.inc"
            : [scbuf] "+s"(scbuf)
            : W4_COMMON_OPERANDS, [eo] "{v[240:243]}"(eo), [sap] "s"(s_sap), [sbp] "s"(s_sbp)
            :
#include "w4_clobbers_i8.inc"
        );
      }
    } else if constexpr (T::DT == DT_BF16) {
      asm volatile(
#include "w4_kloop_bf16.inc"
          : [scbuf] "+s"(scbuf)
          : W4_COMMON_OPERANDS, [eo] "{v[240:243]}"(eo)
          :
#include "w4_clobbers_bf16.inc"
      );
    } else if constexpr (T::DT == DT_F16) {
      asm volatile(
#include "w4_kloop_f16.inc"
          : [scbuf] "+s"(scbuf)
          : W4_COMMON_OPERANDS, [eo] "{v[240:243]}"(eo)
          :
#include "w4_clobbers_f16.inc"
      );
    } else {
      v8i sc;
      sc[0] = (int)(lds0 + 131072u + (uint32_t)(ln.wm0 + ln.r) * 16u + (uint32_t)ln.g * 2u);
      sc[1] = (int)(lds0 + 131072u + (uint32_t)(256 + ln.wn0 + ln.r) * 16u + (uint32_t)ln.g * 2u);
      sc[2] = (int)cur.sca; sc[3] = (int)cur.scb; sc[4] = (int)nxt.sca; sc[5] = (int)nxt.scb; sc[6] = eo[0]; sc[7] = 0;
      const uint8_t *sMa = uniform(cur.mxa), *sMb = uniform(cur.mxb), *sMan = uniform(nxt.mxa), *sMbn = uniform(nxt.mxb);
      asm volatile(
#include "w4_kloop_fp4.inc"
          : [scbuf] "+s"(scbuf)
          : W4_COMMON_OPERANDS, [sc] "{v[232:239]}"(sc), [mxa] "s"(sMa), [mxb] "s"(sMb), [mxan] "s"(sMan), [mxbn] "s"(sMbn)
          :
#include "w4_clobbers_fp4.inc"
      );
    }
#ifdef W4_LAB_TS2
    if (tid == 0 && blockIdx.x < 1024 && ts_n < 31) w4_lab_ts[blockIdx.x * 32 + ts_n] = __builtin_amdgcn_s_memrealtime();
    ++ts_n;
#endif
    bool sk_piece = false;
    if constexpr (SK) {
      if (w.kind == WK_SK_PUBLISH) {
        // not the tile's last piece: publish the partial sums, tagged with this launch's epoch
        sk_piece = true;
        partial_store_w4<T>(p.P + (size_t)sched.sk_id * (256 * 256), wave, lane);
        __builtin_amdgcn_s_waitcnt(0x0070);   // this wave's write-through stores have left the CU
        __syncthreads();                      // ... and so have everybody else's
        if (tid == 0) {
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
          __hip_atomic_store(p.flags + sched.sk_id, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else if (w.kind == WK_SK_OWNER) {
        // the piece that ends the tile: wait for the pieces before it (lower workgroup ids only), add them, store
        sk_piece = true;
        int n = 0, nxt_id = sched.sk_id - 1;
        for (int64_t b = w.seg_begin; b > w.tile_first; b -= sched.q + (nxt_id < sched.rem ? 1 : 0), --nxt_id) ++n;
        if (tid == 0) {
          int ok = 1;
          for (int k = 0; k < n && ok; ++k) {
            uint32_t spins = 0;
            while (__hip_atomic_load(p.flags + (sched.sk_id - 1 - k), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != epoch) {
              if (++spins >= p.spin_limit) { ok = 0; break; }
              __builtin_amdgcn_s_sleep(2);
            }
          }
          s_bcast = ok;
        }
        __syncthreads();
        const bool ok = s_bcast != 0;
        __syncthreads();
        if (!ok) failed = true;
        if (p.c_type == DT_BF16) epilogue_w4_owner<T, DT_BF16>(p, w.tc, ln, wave, lane, sched.sk_id - 1, ok ? n : 0, !ok);
        else if (p.c_type == DT_F16) epilogue_w4_owner<T, DT_F16>(p, w.tc, ln, wave, lane, sched.sk_id - 1, ok ? n : 0, !ok);
        else epilogue_w4_owner<T, DT_F32>(p, w.tc, ln, wave, lane, sched.sk_id - 1, ok ? n : 0, !ok);
      }
    }
    if (sk_piece) {
      fe = 0;
      nst = 0;      // (an unknown number of stores since the K loop)
    } else if (fast && fe_shape && have_next) {
      // stored by the next tile's K loop (2: as fp16)
      fe = p.c_type == DT_F16 ? 2 : 1;
      cprev = (const uint8_t*)p.C + ((int64_t)(w.tc.m0 + ln.wm0) * p.c_sm + (w.tc.n0 + ln.wn0)) * 2;
      nst = 0;
    } else {
      fe = 0;
      // Every workgroup reaches its epilogue at about the same time, so C arrives as bursts of 32 MB; the
      // L2s take such a burst as ordinary write-back lines and drain it behind the next K steps, while
      // non-temporal stores go to the fabric at once and hold the waves at the store queue (measured:
      // FP8 8192x28672x8192 1.24 -> 1.20 ms, MXFP4 8192x8192x16384 0.440 -> 0.415 ms without the hint).
      const bool c_nt = false;
      if (fast) {
        if (p.c_type == DT_BF16) {
          if (c_nt) epilogue_w4_fast<T, DT_BF16, true>(p, w.tc, ln);
          else epilogue_w4_fast<T, DT_BF16, false>(p, w.tc, ln);
        } else {
          if (c_nt) epilogue_w4_fast<T, DT_F16, true>(p, w.tc, ln);
          else epilogue_w4_fast<T, DT_F16, false>(p, w.tc, ln);
        }
      } else if (p.c_type == DT_BF16) epilogue_w4<T, DT_BF16>(p, w.tc, ln);
      else if (p.c_type == DT_F16) epilogue_w4<T, DT_F16>(p, w.tc, ln);
      else if (is_f8(T::DT) && p.c_type == DT_FP8) {
        if constexpr (is_f8(T::DT)) epilogue_w4<T, DT_FP8>(p, w.tc, ln);
      } else if (is_f8(T::DT) && p.c_type == DT_E5M2) {
        if constexpr (is_f8(T::DT)) epilogue_w4<T, DT_E5M2>(p, w.tc, ln);
      } else epilogue_w4<T, DT_F32>(p, w.tc, ln);
      nst = fast ? 1 : 0;
    }
#if defined(W4_LAB_TS) && !defined(W4_LAB_TS2)
    if (tid == 0 && blockIdx.x < 1024 && ts_n < 31) w4_lab_ts[blockIdx.x * 32 + ts_n] = __builtin_amdgcn_s_memrealtime();
    ++ts_n;
#endif
    w = wnext;
    have = have_next;
    first = 0;
  }
  // the last tile's look-ahead copies still write LDS: they must have landed before the workgroup ends
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#ifdef W4_LAB_TS
  if (tid == 0 && blockIdx.x < 1024) w4_lab_ts[blockIdx.x * 32 + 31] = __builtin_amdgcn_s_memrealtime();
#endif
  if constexpr (SK) {
    if (failed && tid == 0) atomicExch(p.ctl + CTL_STATUS, 1u);
    sk_leave(p, epoch, tid);
  }
  if (p.mode == MODE_WS && tid == 0) {
    // the last workgroup to leave rearms the queues for the next launch
    uint32_t done = atomicAdd(p.ctl + CTL_DONE, 1u);
    if (done == gridDim.x - 1) {
      for (int qi = 0; qi <= p.num_xcds * p.counters_per_xcd; ++qi)
        __hip_atomic_store(p.counters + qi * COUNTER_STRIDE, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(p.ctl + CTL_DONE, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace tb
