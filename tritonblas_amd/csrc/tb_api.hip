// C ABI of the library: argument validation, kernel-variant choice and launches.
// No device allocation, no synchronisation, no exceptions: every entry point returns a status.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>
#include "../../include/tritonblas_amd.h"
#include "gemm_variants.h"
#include "quant.h"
#include "skinny.h"
#include "selector.h"

using namespace tb;

// the public element type codes are the kernels' own
static_assert(TB_F16 == DT_F16 && TB_BF16 == DT_BF16 && TB_FP8_E4M3 == DT_FP8 && TB_FP4_E2M1 == DT_FP4 && TB_F32 == DT_F32 &&
              TB_I8 == DT_I8 && TB_FP8_E5M2 == DT_E5M2, "element type codes");

namespace {

constexpr int MAX_DEVICES = 64;
tb_hw g_hw[MAX_DEVICES];
std::once_flag g_hw_once[MAX_DEVICES];
int g_hw_status[MAX_DEVICES];

int read_num_xcc(int n_cu, const char* arch) {
  // KFD reports the XCC count per node; fall back to what the known parts have.
  if (std::strncmp(arch, "gfx950", 6) == 0) return n_cu >= 64 ? std::max(1, n_cu / 32) : 1;
  if (std::strncmp(arch, "gfx942", 6) == 0) {
    if (n_cu == 304) return 8;
    if (n_cu == 228) return 6;
    return std::max(1, n_cu / 38);
  }
  return 1;
}

void query_hw(int dev) {
  hipDeviceProp_t pr;
  if (hipGetDeviceProperties(&pr, dev) != hipSuccess) { g_hw_status[dev] = TB_ERR_NO_DEVICE; return; }
  tb_hw hw;
  default_hw(&hw);
  hw.n_cu = pr.multiProcessorCount;
  std::memset(hw.arch, 0, sizeof(hw.arch));
  for (int i = 0; i < (int)sizeof(hw.arch) - 1 && pr.gcnArchName[i] && pr.gcnArchName[i] != ':'; ++i) hw.arch[i] = pr.gcnArchName[i];
  hw.num_xcd = read_num_xcc(hw.n_cu, hw.arch);
  hw.cu_per_xcd = std::max(1, hw.n_cu / hw.num_xcd);
  hw.lds_bytes = (int)pr.maxSharedMemoryPerMultiProcessor;
  hw.l2_bytes = pr.l2CacheSize;
  hw.clock_khz = pr.clockRate;
  hw.mem_clock_khz = pr.memoryClockRate;
  hw.wave_size = pr.warpSize;
  // HBM3E: bus width (bits) x memory clock x 2 (DDR) / 8; the runtime reports the command clock
  double gbps = (double)pr.memoryBusWidth / 8.0 * (double)pr.memoryClockRate * 1e3 * 2.0 / 1e9;
  hw.hbm_gbps = (gbps > 100.0) ? gbps : 8000.0;
  if (std::strncmp(hw.arch, "gfx950", 6) == 0) hw.hbm_gbps = 8000.0;
  g_hw[dev] = hw;
  g_hw_status[dev] = TB_OK;
}

int current_hw(tb_hw* out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return TB_ERR_NO_DEVICE;
  std::call_once(g_hw_once[dev], query_hw, dev);
  if (g_hw_status[dev] != TB_OK) return g_hw_status[dev];
  *out = g_hw[dev];
  return TB_OK;
}

// Tuning and test hooks.  The TB_* environment variables are read once, when the library first needs
// them; tb_debug_option() changes a hook afterwards (tests switch kernels that way).  Nothing on the
// launch path calls getenv.
struct Hooks {
  int waves = 0;                // TB_WAVES=<wm><wn>[<stages>]: picks among variants that share a tile shape
  int no_mxlds = 0;             // TB_NO_MXLDS=1: fp4 scales straight from global memory (gather kernel)
  int no_cline = 0;             // TB_NO_CLINE=1: element-wise C stores
  int no_skinny = 0, skinny = 0;  // TB_NO_SKINNY / TB_SKINNY: force the small-M kernel choice
  int grid = 0;                 // TB_GRID=<n>: workgroups of a persistent / grouped launch
  int panel = -1;               // TB_PANEL=<n>: column panel width of the tile order (-1: the library's)
  int no_column_split = 0, force_column_split = 0;
  int quant_div64 = 0;          // TB_QUANT_DIV64=1: the quantiser's kernel for 2^31 items and more at any size
  int grp_sk_fix = 0;           // TB_GRP_SK_FIX=<K steps>: what the grouped Stream-K tail's model charges per extra piece of a tile
  int lab = 0;                  // TB_DEBUG=<bits>: 4 = the 4-wave kernels store every tile with their compiled epilogue (none fused
                                // into the next K loop); 1, 2 = only acted on by kernels built with TB_LAB_HOOKS
};
Hooks g_hooks;
std::once_flag g_hooks_once;
std::mutex g_plan_mu;
uint64_t g_hooks_version = 0;   // bumped whenever a hook changes: cached plans are then stale

int env_int(const char* name, int dflt) {
  const char* e = getenv(name);
  return e ? atoi(e) : dflt;
}
void read_hooks() {
  g_hooks.waves = env_int("TB_WAVES", 0);
  g_hooks.no_mxlds = env_int("TB_NO_MXLDS", 0);
  g_hooks.no_cline = env_int("TB_NO_CLINE", 0);
  g_hooks.no_skinny = env_int("TB_NO_SKINNY", 0);
  g_hooks.skinny = env_int("TB_SKINNY", 0);
  g_hooks.grid = env_int("TB_GRID", 0);
  g_hooks.panel = env_int("TB_PANEL", -1);
  g_hooks.no_column_split = env_int("TB_NO_COLUMN_SPLIT", 0);
  g_hooks.force_column_split = env_int("TB_FORCE_COLUMN_SPLIT", 0);
  g_hooks.quant_div64 = env_int("TB_QUANT_DIV64", 0);
  g_hooks.lab = env_int("TB_DEBUG", 0);
  g_hooks.grp_sk_fix = env_int("TB_GRP_SK_FIX", 0);
}
std::mutex g_hooks_mu;
// (a copy taken under the hooks' own lock: tb_debug_option may change one while another thread plans)
Hooks hooks() {
  std::call_once(g_hooks_once, read_hooks);
  std::lock_guard<std::mutex> lk(g_hooks_mu);
  return g_hooks;
}

void variant_table(int dt, const Variant** v, int* n) {
  switch (dt) {
    case TB_F16: *v = g_variants_f16; *n = g_num_variants_f16; break;
    case TB_BF16: *v = g_variants_bf16; *n = g_num_variants_bf16; break;
    case TB_FP8_E4M3: *v = g_variants_fp8; *n = g_num_variants_fp8; break;
    case TB_FP8_E5M2: *v = g_variants_e5m2; *n = g_num_variants_e5m2; break;
    case DT_E4E5: *v = g_variants_e4e5; *n = g_num_variants_e4e5; break;
    case DT_E5E4: *v = g_variants_e5e4; *n = g_num_variants_e5e4; break;
    case TB_FP4_E2M1: *v = g_variants_fp4; *n = g_num_variants_fp4; break;
    case TB_F32: *v = g_variants_f32; *n = g_num_variants_f32; break;
    case TB_I8: *v = g_variants_i8; *n = g_num_variants_i8; break;
    default: *v = nullptr; *n = 0;
  }
}

// distinct tiles (layout-independent) of one element type, fast kernels first
std::vector<TileInfo> tile_infos(int dt) {
  const Variant* v; int n;
  variant_table(dt, &v, &n);
  std::vector<TileInfo> out;
  for (int i = 0; i < n; ++i) {
    bool seen = false;
    for (auto& t : out) seen |= (t.bm == v[i].bm && t.bn == v[i].bn && t.bk == v[i].bk && t.fast == v[i].fast);
    if (!seen) out.push_back(TileInfo{v[i].dt, v[i].bm, v[i].bn, v[i].bk, v[i].threads, v[i].lds_bytes, v[i].minb, v[i].fast, v[i].stages});
  }
  return out;
}

// Variants may share a tile shape and differ in the depth of the copy pipeline.  A deeper pipeline hides
// more of the copy latency of every K step but lets fewer workgroups share a CU, so it only pays while
// all tiles are resident at once: the deepest variant that still holds `total_tiles` on the device is
// taken (measured, 64x64 bf16 tiles: 128x4096x4096 32 -> 22 us, 64x8192x8192 60 -> 39 us with four
// stages; 2048^3 30 -> 35 us, which the rule avoids).
const Variant* find_variant(int dt, int bm, int bn, int bk, int alay, int blay, int fast, int64_t total_tiles = 0,
                            const tb_hw* hw = nullptr, bool need_sk = false, int64_t k = 0, int out8 = 0) {
  const Variant* v; int n;
  variant_table(dt, &v, &n);
  // the hand-scheduled 4-wave kernels run K steps in pairs (the pieces of a Stream-K tail in blocks of four); they
  // store e4m3 results (out8 = 1) from whole tiles only and int8 results (out8 = 2) not at all
  auto usable = [&](const Variant& x) {
    if (!x.k_step_pairs) return true;
    if (out8 == 2 || (out8 == 1 && need_sk) || (need_sk && !x.kernel_sk)) return false;
    return k >= 4 * (int64_t)x.bk && k % ((need_sk ? 4 : 2) * (int64_t)x.bk) == 0;
  };
  const int want = hooks().waves;
  if (want && fast)
    for (int i = 0; i < n; ++i)
      if (usable(v[i]) && v[i].fast == fast && v[i].alay == alay && v[i].blay == blay && v[i].bm == bm && v[i].bn == bn && v[i].bk == bk &&
          (v[i].wm * 10 + v[i].wn == want || v[i].wm * 100 + v[i].wn * 10 + v[i].stages == want))
        return &v[i];
  const Variant* best = nullptr;
  for (int i = 0; i < n; ++i) {
    if (!(usable(v[i]) && v[i].fast == fast && v[i].alay == alay && v[i].blay == blay && (fast == 0 || (v[i].bm == bm && v[i].bn == bn && v[i].bk == bk))))
      continue;
    if (!best) { best = &v[i]; if (!hw || total_tiles <= 0 || !fast) return best; continue; }   // (listed first: the default depth)
    const int occ = std::max(1, std::min(v[i].minb, hw->lds_bytes / std::max(1, v[i].lds_bytes)));
    if (v[i].stages > best->stages && total_tiles <= (int64_t)hw->n_cu * occ) best = &v[i];
  }
  return best;
}

// Width (in tiles) of the column panels of the tile order.  One pass of the grid over the tile list
// ("round") should cover a near-square block of C, so that the A and B strips a round needs are few and
// shared by many workgroups, and the panel's B strips are reused by every row group before they leave
// the memory-side cache.  A multiple of the width of one XCD's block (chunk / group_m columns).
int default_panel_n(int grid, int chunk, int group_m) {
  const int bw = std::max(1, chunk / std::max(1, group_m));
  int side = 1;
  while (side * side < grid) ++side;
  return std::max(bw, (side + bw - 1) / bw * bw);
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }
int unit_bytes(int dt) { return (dt == TB_F16 || dt == TB_BF16) ? 2 : (dt == TB_F32 ? 4 : 1); }
bool is_f8_type(int t) { return t == TB_FP8_E4M3 || t == TB_FP8_E5M2; }
// The kernels' element type code for a pair of operand types: the type itself when both agree, the codes of the two
// mixtures of 8-bit float formats (reference origami.py:98-112 and matmul.py:42-66 take the two types separately), -1 for
// any other pair.
int kernel_type(int a_type, int b_type) {
  if (a_type == b_type) return a_type;
  if (a_type == TB_FP8_E4M3 && b_type == TB_FP8_E5M2) return DT_E4E5;
  if (a_type == TB_FP8_E5M2 && b_type == TB_FP8_E4M3) return DT_E5E4;
  return -1;
}
// the type the cost model prices a kernel type as (the mixtures run the e5m2 kernels' instruction stream)
int model_type(int dt) { return (dt == DT_E4E5 || dt == DT_E5E4) ? TB_FP8_E5M2 : dt; }
int c_bytes(int t) { return t == TB_F32 ? 4 : ((t == TB_I8 || is_f8_type(t)) ? 1 : 2); }

// Everything the launch path needs, independent of which public descriptor it came from.
struct Job {
  int dt = 0, c_type = 0, bias_type = 0;
  int64_t M = 0, N = 0, K = 0;
  const void* A = nullptr; const void* B = nullptr; void* C = nullptr;
  int64_t a_sr = 0, a_sk = 0, b_sr = 0, b_sk = 0;  // storage units: row = m (A) / n (B)
  int64_t c_sm = 0, c_sn = 0;
  const float* sa = nullptr; const float* sb = nullptr;
  const void* bias = nullptr; int64_t bias_stride = 0;
  const void* mxa = nullptr; const void* mxb = nullptr;
  int64_t mxa_sr = 0, mxa_sk = 0, mxb_sr = 0, mxb_sk = 0;
  int bm = 0, bn = 0, bk = 0, group_m = 0, num_xcds = 0;
  int schedule = TB_SCHED_PERSISTENT, grid = 0, counters_per_xcd = 0;
  void* workspace = nullptr; size_t workspace_bytes = 0;
  uint32_t epoch = 1, spin_limit = 0;
  const int32_t* cu_mask = nullptr; int cu_mask_len = 0, ws_mode = 0, ws_local = 0, ws_global = 0;
  // grouped
  const int32_t* group_offsets = nullptr; int num_groups = 0;
  int64_t b_group_stride = 0, sb_group_stride = 0;
  int grp_phase = 0, grp_big = 0, grp_thr = 0, grp_auto = 0;   // see GemmParams
  int grp_sk = 0;          // grouped: cut the tiles that do not fill whole rounds of the grid into K ranges (needs a workspace)
  int column_split = 0;
};

// Workspace layout (bytes): [0, 256) control words | work-stealing queue counters, one 256-byte line
// each, WS_MAX_LINES lines | Stream-K flags, one word per workgroup | Stream-K partial tiles.  The
// regions never overlap whatever schedule a launch runs, so one workspace serves Stream-K launches
// (whose flags are never cleared: they carry epochs) and work-stealing launches (whose counters must
// be zero when a launch starts) in any order.
constexpr size_t WS_MAX_LINES = 520;   // 8 XCDs x 64 slots, a shared pool, spare
constexpr size_t WS_COUNTERS_OFF = CTL_WORDS * 4;
constexpr size_t WS_FLAGS_OFF = WS_COUNTERS_OFF + WS_MAX_LINES * COUNTER_STRIDE * 4;

struct Plan {
  const Variant* v = nullptr;
  GemmParams p;
  int grid = 0;
  bool skinny = false;   // decode shapes: streaming kernel without tiles or workspace
  size_t ws_need = 0, ws_flags_off = 0, ws_p_off = 0, ws_counters_off = 0;
};

bool is_streamk(int schedule) { return schedule == TB_SCHED_STREAMK || schedule == TB_SCHED_STREAMK_WS; }

int kernel_occupancy(const Variant* v, const void* kernel) {
  static std::mutex mu;
  static std::vector<std::pair<const void*, int>> cache;
  std::lock_guard<std::mutex> lk(mu);
  for (auto& c : cache) if (c.first == kernel) return c.second;
  int nb = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, kernel, v->threads, 0) != hipSuccess || nb < 1) nb = 1;
  cache.emplace_back(kernel, nb);
  return nb;
}

int make_plan(const Job& j, const tb_hw& hw, bool need_device, Plan* plan) {
  if (j.M <= 0 || j.N <= 0 || j.K <= 0) return TB_ERR_BAD_SHAPE;
  if (j.M > INT32_MAX || j.N > INT32_MAX) return TB_ERR_BAD_SHAPE;
  if (j.c_type != TB_F16 && j.c_type != TB_BF16 && j.c_type != TB_F32 && !(j.c_type == TB_I8 && j.dt == TB_I8) &&
      !(is_f8_type(j.c_type) && is_f8(j.dt)))
    return TB_ERR_BAD_DTYPE;
  const int usz = unit_bytes(j.dt);
  const int epu = (j.dt == TB_FP4_E2M1) ? 2 : 1;
  if (j.K % epu) return TB_ERR_BAD_SHAPE;
  const int64_t KU = j.K / epu;

  // which loader can address each operand
  auto k_major_ok = [&](const void* ptr, int64_t s_row, int64_t s_k, int64_t rows) {
    return s_k == 1 && aligned16(ptr) && (rows == 1 || (s_row * usz) % 16 == 0) && s_row >= 0;
  };
  auto m_major_ok = [&](const void* ptr, int64_t s_row, int64_t s_k, int64_t rows) {
    return usz == 2 && s_row == 1 && aligned16(ptr) && (s_k * usz) % 16 == 0 && rows % 8 == 0 && j.num_groups == 0;
  };
  int alay = -1, blay = -1;
  if (k_major_ok(j.A, j.a_sr, j.a_sk, j.M)) alay = LAY_K; else if (m_major_ok(j.A, j.a_sr, j.a_sk, j.M)) alay = LAY_M;
  if (k_major_ok(j.B, j.b_sr, j.b_sk, j.N)) blay = LAY_K; else if (m_major_ok(j.B, j.b_sr, j.b_sk, j.N)) blay = LAY_M;

  // tile
  int bm = j.bm, bn = j.bn, bk = j.bk;
  tb_selection sel;
  std::memset(&sel, 0, sizeof(sel));
  if (bm == 0 || bn == 0 || bk == 0) {
    tb_problem pr;
    std::memset(&pr, 0, sizeof(pr));
    pr.m = j.M; pr.n = j.N; pr.k = j.K; pr.a_type = pr.b_type = model_type(j.dt); pr.c_type = j.c_type;
    pr.a_k_contiguous = alay == LAY_K; pr.b_k_contiguous = blay == LAY_K;
    pr.streamk = is_streamk(j.schedule); pr.num_groups = j.num_groups;
    auto infos = tile_infos(j.dt);
    int st = select_tile(pr, hw, infos.data(), (int)infos.size(), &sel);
    if (st != TB_OK) return st;
    bm = sel.block_m; bn = sel.block_n; bk = sel.block_k;
  }
  const Variant* v = nullptr;
  bool fast = alay >= 0 && blay >= 0 && (KU % (bk / epu) == 0);
  if (j.dt == TB_FP4_E2M1) {
    // the fast fp4 kernels stage 16 scale bytes per row at a time through LDS with 16-byte copies
    const bool mx_ok = j.mxa_sk == 1 && j.mxb_sk == 1 && (j.K / 32) % 16 == 0 && j.mxa_sr % 16 == 0 && j.mxb_sr % 16 == 0 &&
                       ((uintptr_t)j.mxa % 16) == 0 && ((uintptr_t)j.mxb % 16) == 0;
    if (!mx_ok || hooks().no_mxlds) fast = false;
  }
  if (fast) {
    // 32-bit offsets inside a tile
    if ((alay == LAY_K && (int64_t)bm * j.a_sr * usz >= (1ll << 31)) || (blay == LAY_K && (int64_t)bn * j.b_sr * usz >= (1ll << 31)) ||
        (alay == LAY_M && (int64_t)bk * j.a_sk * usz >= (1ll << 31)) || (blay == LAY_M && (int64_t)bk * j.b_sk * usz >= (1ll << 31)))
      fast = false;
  }
  if (fast) {
    // workgroups that have to be resident at once for a deeper-pipeline variant to be the better one:
    // all tiles, and for Stream-K the whole grid (the owners wait for the other segments' workgroups)
    int64_t at_once = ((j.M + bm - 1) / bm) * ((j.N + bn - 1) / bn);
    if (is_streamk(j.schedule)) at_once = j.grid > 0 ? std::max<int64_t>(at_once, j.grid) : 0;
    if (j.num_groups > 0) at_once = 0;
    v = find_variant(j.dt, bm, bn, bk, alay, blay, 1, at_once, &hw, is_streamk(j.schedule) && j.num_groups == 0, j.K,
                     j.c_type == TB_I8 ? 2 : (is_f8_type(j.c_type) ? 1 : 0));
    if (!v) return TB_ERR_BAD_TILE;
  } else {
    if (j.bm != 0) {
      // an explicit tile must at least name a built one, even when the gather kernel runs instead
      bool known = false;
      for (auto& t : tile_infos(j.dt)) known |= (t.bm == bm && t.bn == bn && t.bk == bk);
      if (!known) return TB_ERR_BAD_TILE;
    }
    v = find_variant(j.dt, 0, 0, 0, LAY_K, LAY_K, 0);
    if (!v) return TB_ERR_BAD_LAYOUT;
  }
  if (j.dt == TB_FP4_E2M1 && (j.a_sk != 1 || j.b_sk != 1)) return TB_ERR_BAD_LAYOUT;

  GemmParams& p = plan->p;
  std::memset(&p, 0, sizeof(p));
  p.A = (const uint8_t*)j.A; p.B = (const uint8_t*)j.B; p.C = (uint8_t*)j.C;
  p.sa = j.sa; p.sb = j.sb; p.bias = (const uint8_t*)j.bias;
  p.mxa = (const uint8_t*)j.mxa; p.mxb = (const uint8_t*)j.mxb;
  p.M = (int32_t)j.M; p.N = (int32_t)j.N; p.KU = KU;
  p.a_sr = j.a_sr; p.a_sk = j.a_sk; p.b_sr = j.b_sr; p.b_sk = j.b_sk;
  p.c_sm = j.c_sm; p.c_sn = j.c_sn;
  p.mxa_sr = j.mxa_sr; p.mxa_sk = j.mxa_sk; p.mxb_sr = j.mxb_sr; p.mxb_sk = j.mxb_sk;
  p.bias_stride = j.bias_stride; p.c_type = j.c_type; p.bias_type = j.bias_type;
  p.a_vec = p.b_vec = v->fast;
  const int cb = c_bytes(j.c_type);
  p.c_vec = (j.c_sn == 1 && (j.c_sm % 4 == 0 || j.M == 1) && ((uintptr_t)j.C % (4 * cb)) == 0) ? 1 : 0;
  p.c_line = (j.c_type != TB_I8 && !is_f8_type(j.c_type) && j.c_sn == 1 && ((j.c_sm * cb) % 16 == 0 || j.M == 1) && ((uintptr_t)j.C % 16) == 0) ? 1 : 0;
  if (hooks().no_cline) p.c_line = 0;
  // (8192x28672x8192 FP8 +0.6 %, 8192^3 bf16 +1.6 %; a small C stays cacheable for whoever reads it next)
  p.c_nt = ((int64_t)j.M * j.N * cb > (int64_t)hw.num_xcd * std::max(hw.l2_bytes, 1 << 20)) ? 1 : 0;
  if (j.dt == TB_FP4_E2M1) {
    const int ksub = v->bk / 128;
    p.mx_vec = (j.mxa_sk == 1 && j.mxb_sk == 1 && j.mxa_sr % ksub == 0 && j.mxb_sr % ksub == 0 &&
                ((uintptr_t)j.mxa % ksub) == 0 && ((uintptr_t)j.mxb % ksub) == 0) ? 1 : 0;
    p.mx_lds = v->fast;
  }
  p.tiles_m = (int32_t)((j.M + v->bm - 1) / v->bm);
  p.tiles_n = (int32_t)((j.N + v->bn - 1) / v->bn);
  const int64_t total = (int64_t)p.tiles_m * p.tiles_n;
  if (total > INT32_MAX) return TB_ERR_BAD_SHAPE;
  p.total_tiles = (int32_t)total;
  p.k_iters = (int32_t)((j.K + v->bk - 1) / v->bk);
  p.group_m = j.group_m > 0 ? j.group_m : std::min(8, (int)p.tiles_m);
  p.num_xcds = j.num_xcds > 0 ? j.num_xcds : hw.num_xcd;
  p.epoch = j.epoch; p.spin_limit = j.spin_limit ? j.spin_limit : (1u << 24);
  p.debug = hooks().lab;
  p.group_offsets = j.group_offsets; p.num_groups = j.num_groups;
  p.b_group_stride = j.b_group_stride; p.sb_group_stride = j.sb_group_stride;

  const void* kern = (is_streamk(j.schedule) && j.num_groups == 0) ? v->kernel_sk : v->kernel;
  {
    // a handful of rows against a K-major weight: the streaming kernel (no tiles, no workspace) when
    // the model expects it to beat the tile kernel of the requested schedule.  TB_NO_SKINNY=1 / TB_SKINNY=1
    // force the choice (tuning and tests).
    plan->skinny = j.num_groups == 0 && skinny_supported(j.dt, j.M) && alay == LAY_K && blay == LAY_K &&
                   KU % skinny_k_step_units(j.dt) == 0 && j.N >= 1024 && !hooks().no_skinny && !is_f8_type(j.c_type);
    if (plan->skinny && !hooks().skinny) {
      tb_problem pr;
      std::memset(&pr, 0, sizeof(pr));
      pr.m = j.M; pr.n = j.N; pr.k = j.K; pr.a_type = pr.b_type = model_type(j.dt); pr.c_type = j.c_type;
      pr.a_k_contiguous = pr.b_k_contiguous = 1;
      const bool sk = is_streamk(j.schedule);
      const TileInfo ti{v->dt, v->bm, v->bn, v->bk, v->threads, v->lds_bytes, v->minb, v->fast, v->stages};
      plan->skinny = estimate_streaming_us(pr, hw) < estimate_tile_us(pr, hw, ti, sk);
    }
    if (plan->skinny) { plan->v = v; plan->grid = 1; plan->ws_need = 0; return TB_OK; }
  }
  const int occ = need_device ? kernel_occupancy(v, kern) : std::max(1, std::min(v->minb, hw.lds_bytes / v->lds_bytes));
  const int resident = hw.n_cu * occ;
  int grid;
  plan->ws_need = 0;
  if (j.num_groups > 0) {
    // the tile table has at most this many entries (every expert may end in a partial row block);
    // a resident grid loops over it
    p.mode = MODE_GROUPED;
    p.grp_phase = j.grp_phase; p.grp_big = j.grp_big; p.grp_thr = j.grp_thr; p.grp_auto = j.grp_auto;
    if (p.grp_phase == 1) {
      // only a tall fast tile leaves its short last blocks to a second launch
      if (v->fast && v->bm >= 128 && j.grp_thr > 0 && j.grp_thr < v->bm) p.grp_big = v->bm;
      else p.grp_phase = 0;
    }
    if (p.grp_phase == 2 && (p.grp_big <= 0 || p.grp_thr <= 0)) return TB_ERR_BAD_ARGUMENT;
    const int64_t bound = p.grp_phase == 2
        ? (int64_t)j.num_groups * ((j.grp_thr + v->bm - 1) / v->bm) * p.tiles_n
        : ((j.M + v->bm - 1) / v->bm + j.num_groups) * p.tiles_n;
    if (bound > INT32_MAX) return TB_ERR_BAD_SHAPE;
    p.total_tiles = (int32_t)bound;
    grid = (int)std::min<int64_t>(bound, resident);
    if (hooks().grid > 0) grid = (int)std::min<int64_t>(bound, hooks().grid);
    // Stream-K tail: only the hand-scheduled 4-wave kernel has the cheap exchange of partial tiles that makes
    // it pay (K ranges in blocks of four steps), and only the launch of the tall tiles
    if (j.grp_sk && p.grp_phase != 2 && v->k_step_pairs && v->kernel_sk && p.k_iters % 4 == 0 && p.k_iters >= 8 && occ == 1) {
      p.grp_sk = 1;
      // (measured with 8 experts, 2072 tiles of 32 K steps on 256 workgroups: the launch that cuts 280 tiles
      // takes 63 us longer than 7 whole rounds and 35 K steps would -- every workgroup writes and reads a
      // 256 KB partial tile while the operand strips already keep the fabric busy -- i.e. about 48 K steps, and
      // the kernel that can cut is 12 us slower than the one that cannot even when it cuts nothing)
      p.grp_sk_fix = hooks().grp_sk_fix > 0 ? hooks().grp_sk_fix : 64;
      p.sk_unit = 4;
      plan->ws_flags_off = WS_FLAGS_OFF;
      plan->ws_p_off = plan->ws_flags_off + (((size_t)grid * 4 + 255) / 256) * 256;
      plan->ws_need = plan->ws_p_off + (size_t)grid * v->bm * v->bn * 4;
    }
  } else if (j.schedule == TB_SCHED_PERSISTENT) {
    // a resident grid that loops over the tiles (matmul.py:160-198: for tile_id in range(pid, total, NUM_SMS))
    p.mode = MODE_STATIC;
    grid = (int)std::min<int64_t>(total, j.grid > 0 ? j.grid : resident);
    if (hooks().grid > 0) grid = (int)std::min<int64_t>(total, hooks().grid);
  } else if (j.schedule == TB_SCHED_WORK_STEALING) {
    p.mode = MODE_WS;
    grid = j.grid > 0 ? j.grid : (j.cu_mask ? j.cu_mask_len : resident);
    if (j.cu_mask && (j.cu_mask_len <= 0 || grid > j.cu_mask_len)) return TB_ERR_BAD_ARGUMENT;
    p.cu_mask = j.cu_mask;
    p.counters_per_xcd = j.counters_per_xcd > 0 ? j.counters_per_xcd : ws_counters_per_xcd(total);
    p.ws_mode = j.ws_mode;
    if (j.ws_mode == TB_WS_HIERARCHICAL) {
      int64_t local = j.ws_local, global = j.ws_global;
      if (local == 0 && global == 0) hierarchical_split(total, hw.num_xcd * hw.cu_per_xcd, p.num_xcds, &local, &global);
      if (local < 0 || global < 0 || local * p.num_xcds + global != total) return TB_ERR_BAD_SCHEDULE;
      p.ws_local = (int32_t)local; p.ws_global = (int32_t)global;
    } else if (j.ws_mode != TB_WS_QUEUES && j.ws_mode != TB_WS_GLOBAL_ATOMIC) {
      return TB_ERR_BAD_SCHEDULE;
    }
    // one counter line per XCD x slot, plus the line of the hierarchical mode's shared pool
    if ((size_t)p.num_xcds * p.counters_per_xcd + 1 > WS_MAX_LINES) return TB_ERR_BAD_SCHEDULE;
    plan->ws_counters_off = WS_COUNTERS_OFF;
    plan->ws_need = WS_FLAGS_OFF;
  } else if (is_streamk(j.schedule)) {
    p.mode = MODE_SK;
    p.sk_unit = v->k_step_pairs ? 4 : 1;
    // (a requested grid larger than what is resident at once for the kernel that really runs -- the caller
    // sized it for another tile, e.g. the operands turned out to need the gather kernel -- gives way to
    // the library's own choice.  Correctness does not need residency: a tile's owner only waits for
    // workgroups with lower ids, which the hardware has started before it.  But an owner that waits
    // occupies its CU, so a grid beyond residency only adds waiting.)
    int64_t g = j.grid;
    if (g <= 0 || g > resident) {
      tb_problem pr;
      std::memset(&pr, 0, sizeof(pr));
      pr.m = j.M; pr.n = j.N; pr.k = j.K; pr.a_type = pr.b_type = model_type(j.dt); pr.c_type = j.c_type;
      pr.a_k_contiguous = pr.b_k_contiguous = 1; pr.streamk = 1;
      tb_hw hw_res = hw;   // (what the model may fill: the kernel's real occupancy)
      const TileInfo ti{v->dt, v->bm, v->bn, v->bk, v->threads, v->lds_bytes, occ, v->fast, v->stages};
      g = streamk_grid_for(pr, hw_res, ti);
      // (the model's "whole tiles only" answer is the tile count itself and must survive the clamp)
      if (g >= total) g = total;
      else if (g > resident) g = resident;
    }
    const bool whole_only = g == total;   // exactly one workgroup per tile (however many fit at once): nothing to share
    if (whole_only) g = std::min<int64_t>(total, resident);
    if (g > resident) return TB_ERR_BAD_SCHEDULE;
    grid = (int)g;
    p.sk_tiles = whole_only ? 0 : (int32_t)(total % grid);
    if (p.sk_tiles == 0) {
      // nothing to share: the same tiles on the whole-tile kernel (identical results, no workspace) --
      // which may be the hand-scheduled 4-wave form of this tile, ruled out above only for its lack of
      // a Stream-K tail (same tile, one workgroup per CU either way, bit-identical sums)
      p.mode = MODE_STATIC;
      p.sk_unit = 0;
      if (j.schedule == TB_SCHED_STREAMK_WS) {
        // (the work-stealing launch of the same tiles; its workspace is the queue counters)
        Job whole = j;
        whole.schedule = TB_SCHED_WORK_STEALING;
        whole.grid = 0;
        return make_plan(whole, hw, need_device, plan);
      }
      if (v->fast && j.c_type != TB_I8) {
        const Variant* w = find_variant(j.dt, v->bm, v->bn, v->bk, v->alay, v->blay, 1, 0, &hw, false, j.K, is_f8_type(j.c_type) ? 1 : 0);
        if (w && w->k_step_pairs && w->bm == v->bm && w->bn == v->bn && w->bk == v->bk &&
            std::max(1, std::min(w->minb, hw.lds_bytes / w->lds_bytes)) == occ)
          v = w;
      }
    } else {
      plan->ws_flags_off = WS_FLAGS_OFF;
      plan->ws_p_off = plan->ws_flags_off + (((size_t)grid * 4 + 255) / 256) * 256;
      plan->ws_need = plan->ws_p_off + (size_t)grid * v->bm * v->bn * 4;
      if (j.schedule == TB_SCHED_STREAMK_WS) {
        // the whole tiles in front of the tail come from the XCD x slot queues (counters and flags never overlap)
        p.sk_ws = 1;
        p.counters_per_xcd = j.counters_per_xcd > 0 ? j.counters_per_xcd : ws_counters_per_xcd(total - p.sk_tiles);
        if ((size_t)p.num_xcds * p.counters_per_xcd + 1 > WS_MAX_LINES) return TB_ERR_BAD_SCHEDULE;
        plan->ws_counters_off = WS_COUNTERS_OFF;
      }
    }
  } else {
    return TB_ERR_BAD_SCHEDULE;
  }
  if (grid <= 0) return TB_ERR_BAD_SHAPE;
  p.chunk = std::min(p.group_m * p.group_m, std::max(1, grid / p.num_xcds));
  p.panel_n = default_panel_n(grid, p.chunk, p.group_m);
  if (hooks().panel >= 0) p.panel_n = hooks().panel;
  plan->grid = grid;
  plan->v = v;
  return TB_OK;
}

int run_plan(const Job& j, Plan& plan, hipStream_t stream);

// ---- plan cache ------------------------------------------------------------------------------------
// A plan (kernel variant, grid, tile order, schedule parameters) depends on the sizes, strides, types
// and options of a job and on the alignment of its pointers, not on the pointers themselves.  The
// launch path keeps the last plans it made and only refreshes the pointers, so a repeated call does not
// score tiles again (a persistent tb_gemm that considers a column split makes three plans and prices
// two sub-problems).
struct PlanKey {
  int64_t v[56];
  bool operator==(const PlanKey& o) const { return std::memcmp(v, o.v, sizeof(v)) == 0; }
};
// (every field in a slot of its own: packed fields of a descriptor with a negative or oversized value would
// overlap and let one job find another job's plan, or its cached error)
PlanKey plan_key(const Job& j, int dev) {
  PlanKey k;
  std::memset(&k, 0, sizeof(k));
  auto al = [](const void* q) { return (int64_t)((uintptr_t)q & 255) | (q ? 256 : 0); };
  int i = 0;
  const int64_t f[] = {
      j.dt, j.c_type, j.bias_type, j.schedule, dev, j.M, j.N, j.K, j.a_sr, j.a_sk, j.b_sr, j.b_sk, j.c_sm, j.c_sn,
      j.mxa_sr, j.mxa_sk, j.mxb_sr, j.mxb_sk, j.bias_stride, j.bm, j.bn, j.bk, j.group_m, j.num_xcds, j.grid,
      j.counters_per_xcd, j.ws_mode, j.ws_local, j.cu_mask_len, j.ws_global, j.num_groups, j.grp_phase, j.grp_big,
      j.grp_thr, j.grp_auto, j.grp_sk, j.b_group_stride, j.sb_group_stride, al(j.A), al(j.B), al(j.C), al(j.mxa), al(j.mxb),
      al(j.bias), j.sa ? 1 : 0, j.sb ? 1 : 0, j.cu_mask ? 1 : 0, j.group_offsets ? 1 : 0, j.column_split,
      (int64_t)g_hooks_version};
  static_assert(sizeof(f) <= sizeof(k.v), "PlanKey too small");
  for (int64_t x : f) k.v[i++] = x;
  return k;
}
// the fields of a plan that name memory or change from call to call
void refresh_plan(const Job& j, Plan* plan) {
  GemmParams& p = plan->p;
  p.A = (const uint8_t*)j.A; p.B = (const uint8_t*)j.B; p.C = (uint8_t*)j.C;
  p.sa = j.sa; p.sb = j.sb; p.bias = (const uint8_t*)j.bias;
  p.mxa = (const uint8_t*)j.mxa; p.mxb = (const uint8_t*)j.mxb;
  p.group_offsets = j.group_offsets;
  p.cu_mask = (p.mode == MODE_WS) ? j.cu_mask : nullptr;
  p.epoch = j.epoch; p.spin_limit = j.spin_limit ? j.spin_limit : (1u << 24);
}
struct CachedPlan { PlanKey key; Plan plan; int status; uint64_t stamp; };
constexpr int PLAN_CACHE = 32;
CachedPlan g_plans[PLAN_CACHE];
int g_plans_used = 0;
uint64_t g_plan_clock = 0;

int cached_plan(const Job& j, const tb_hw& hw, Plan* out) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  std::lock_guard<std::mutex> lk(g_plan_mu);
  const PlanKey key = plan_key(j, dev);
  for (int i = 0; i < g_plans_used; ++i)
    if (g_plans[i].key == key) {
      g_plans[i].stamp = ++g_plan_clock;
      if (g_plans[i].status != TB_OK) return g_plans[i].status;
      *out = g_plans[i].plan;
      refresh_plan(j, out);
      return TB_OK;
    }
  Plan plan;
  const int st = make_plan(j, hw, true, &plan);
  int slot = g_plans_used;
  if (g_plans_used < PLAN_CACHE) ++g_plans_used;
  else {
    slot = 0;
    for (int i = 1; i < PLAN_CACHE; ++i) if (g_plans[i].stamp < g_plans[slot].stamp) slot = i;
  }
  g_plans[slot].key = key; g_plans[slot].plan = plan; g_plans[slot].status = st; g_plans[slot].stamp = ++g_plan_clock;
  if (st == TB_OK) *out = plan;
  return st;
}

int launch(const Job& j, hipStream_t stream) {
  tb_hw hw;
  int st = current_hw(&hw);
  if (st != TB_OK) return st;
  Plan plan;
  st = cached_plan(j, hw, &plan);
  if (st != TB_OK) return st;
  return run_plan(j, plan, stream);
}

int run_plan(const Job& j, Plan& plan, hipStream_t stream) {
  GemmParams& p = plan.p;
  if (plan.skinny) {
    if (launch_skinny(p, j.dt, stream) != hipSuccess) { (void)hipGetLastError(); return TB_ERR_LAUNCH; }
    return TB_OK;
  }
  if (plan.ws_need) {
    if (!j.workspace || j.workspace_bytes < plan.ws_need || ((uintptr_t)j.workspace & 255)) return TB_ERR_WORKSPACE;
    // Stream-K flags carry the launch epoch and are never cleared: epoch 0 is what a fresh, zeroed
    // workspace holds in every flag, so a launch tagged 0 would take unpublished partial tiles for published
    if ((p.mode == MODE_SK || p.grp_sk) && j.epoch == 0) return TB_ERR_BAD_ARGUMENT;
    uint8_t* ws = (uint8_t*)j.workspace;
    p.ctl = (uint32_t*)ws;
    if (p.mode == MODE_WS || p.sk_ws) p.counters = (int32_t*)(ws + plan.ws_counters_off);
    if (p.mode == MODE_SK || p.grp_sk) { p.flags = (uint32_t*)(ws + plan.ws_flags_off); p.P = (float*)(ws + plan.ws_p_off); }
  }
  void* args[] = {(void*)&p};
  const void* kern = (p.mode == MODE_SK || p.grp_sk) ? plan.v->kernel_sk : plan.v->kernel;
  hipError_t e = hipLaunchKernel(kern, dim3((unsigned)plan.grid), dim3((unsigned)plan.v->threads), args, 0, stream);
  if (e != hipSuccess) { (void)hipGetLastError(); return TB_ERR_LAUNCH; }
  return TB_OK;
}

// Persistent schedule with a partial last round: a resident grid of G workgroups needs ceil(tiles / G)
// rounds however few tiles the last one holds.  When the model expects it to pay, the columns that fill
// whole rounds run with the planned tile and the remaining columns as a problem of their own, with the
// tile the model picks for them (usually a smaller one that spreads over all CUs).  Both launches write
// disjoint column ranges of C on the same stream.
struct SplitChoice { PlanKey key; int64_t n1; uint64_t stamp; };   // n1 = 0: one launch
SplitChoice g_splits[PLAN_CACHE];
int g_splits_used = 0;

// columns [0, n1) keep the planned tile, the rest becomes a problem of its own; 0 = do not split
int64_t column_split_point(const Job& j, const tb_hw& hw, const Plan& whole) {
  const Variant* v = whole.v;
  const int64_t total = whole.p.total_tiles, G = whole.grid, tiles_m = whole.p.tiles_m, tiles_n = whole.p.tiles_n;
  if (whole.skinny || whole.p.mode != MODE_STATIC || !v->fast || total <= G || total % G == 0) return 0;
  const int64_t tn1 = (total / G) * G / tiles_m;
  if (tn1 <= 0 || tn1 >= tiles_n) return 0;
  const int64_t n1 = tn1 * v->bn, n2 = j.N - n1;
  tb_problem pr;
  std::memset(&pr, 0, sizeof(pr));
  pr.m = j.M; pr.n = j.N; pr.k = j.K; pr.a_type = pr.b_type = model_type(j.dt); pr.c_type = j.c_type;
  pr.a_k_contiguous = pr.b_k_contiguous = 1;
  const TileInfo ti{v->dt, v->bm, v->bn, v->bk, v->threads, v->lds_bytes, v->minb, v->fast, v->stages};
  const double t_whole = estimate_tile_us(pr, hw, ti, false);
  pr.n = n1;
  const double t_first = estimate_tile_us(pr, hw, ti, false);
  pr.n = n2;
  tb_selection rest;
  auto infos = tile_infos(j.dt);
  if (select_tile(pr, hw, infos.data(), (int)infos.size(), &rest) != TB_OK) return 0;
  // (testing hook: TB_FORCE_COLUMN_SPLIT=1 splits whatever the model says)
  if (!hooks().force_column_split && t_first + rest.est_total_us > 0.97 * t_whole) return 0;
  return n1;
}

int launch_columns(const Job& j, hipStream_t stream) {
  if (j.schedule == TB_SCHED_STREAMK && j.column_split == 0 && j.num_groups == 0 && !hooks().no_column_split) {
    // A Stream-K launch whose plan shares no tile runs whole tiles on the whole-tile kernel; it is then the
    // persistent launch of the same tile, partial last round and all, and is treated as one.
    tb_hw hw;
    int st = current_hw(&hw);
    if (st != TB_OK) return st;
    Plan plan;
    st = cached_plan(j, hw, &plan);
    if (st != TB_OK) return st;
    if (plan.skinny || plan.p.mode != MODE_STATIC) return run_plan(j, plan, stream);
    Job whole = j;
    whole.schedule = TB_SCHED_PERSISTENT;
    whole.grid = 0;
    whole.bm = plan.v->bm; whole.bn = plan.v->bn; whole.bk = plan.v->bk;
    whole.workspace = nullptr; whole.workspace_bytes = 0;
    return launch_columns(whole, stream);
  }
  if (j.schedule != TB_SCHED_PERSISTENT || j.column_split != 0 || j.grid > 0 || j.num_groups > 0 || hooks().no_column_split)
    return launch(j, stream);
  tb_hw hw;
  int st = current_hw(&hw);
  if (st != TB_OK) return st;
  Plan whole;
  st = cached_plan(j, hw, &whole);
  if (st != TB_OK) return st;
  int dev = 0;
  (void)hipGetDevice(&dev);
  int64_t n1 = -1;
  {
    std::lock_guard<std::mutex> lk(g_plan_mu);
    const PlanKey key = plan_key(j, dev);
    for (int i = 0; i < g_splits_used && n1 < 0; ++i)
      if (g_splits[i].key == key) { n1 = g_splits[i].n1; g_splits[i].stamp = ++g_plan_clock; }
    if (n1 < 0) {
      n1 = column_split_point(j, hw, whole);
      int slot = g_splits_used;
      if (g_splits_used < PLAN_CACHE) ++g_splits_used;
      else {
        slot = 0;
        for (int i = 1; i < PLAN_CACHE; ++i) if (g_splits[i].stamp < g_splits[slot].stamp) slot = i;
      }
      g_splits[slot].key = key; g_splits[slot].n1 = n1; g_splits[slot].stamp = ++g_plan_clock;
    }
  }
  if (n1 <= 0) return run_plan(j, whole, stream);
  const Variant* v = whole.v;
  const int usz = unit_bytes(j.dt);
  Job a = j, b = j;
  a.N = n1; a.bm = v->bm; a.bn = v->bn; a.bk = v->bk;
  b.N = j.N - n1; b.bm = b.bn = b.bk = 0; b.group_m = 0;
  b.B = (const uint8_t*)j.B + n1 * j.b_sr * usz;
  b.C = (uint8_t*)j.C + n1 * j.c_sn * c_bytes(j.c_type);
  if (j.sb) b.sb = j.sb + n1;
  if (j.bias) b.bias = (const uint8_t*)j.bias + n1 * j.bias_stride * (j.bias_type == TB_F32 ? 4 : 2);
  if (j.mxb) b.mxb = (const uint8_t*)j.mxb + n1 * j.mxb_sr;
  Plan pa, pb;
  st = cached_plan(a, hw, &pa);
  if (st == TB_OK) st = cached_plan(b, hw, &pb);
  if (st != TB_OK || pa.v != v) return run_plan(j, whole, stream);   // (the split must not change what the main part runs)
  st = run_plan(a, pa, stream);
  if (st != TB_OK) return st;
  return run_plan(b, pb, stream);
}

// ---- the library's own scratch buffer ---------------------------------------------------------------
// tb_gemm_static_workspace() runs the schedules that need a workspace without one from the caller: the
// queue counters, Stream-K flags and partial tiles live in this array.  Each device holds its own copy
// at its own address; the array's name is only a handle for hipGetSymbolAddress in host code.
constexpr size_t SCRATCH_BYTES = TB_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

struct ScratchState {
  void* ptr = nullptr;
  int status = TB_ERR_NO_DEVICE;
};
ScratchState g_scratch[MAX_DEVICES];
std::once_flag g_scratch_once[MAX_DEVICES];

void init_scratch(int dev) {
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));   // (the current device's copy)
  if (e != hipSuccess || !ptr) { (void)hipGetLastError(); g_scratch[dev].status = TB_ERR_NO_DEVICE; return; }
  g_scratch[dev].ptr = ptr;
  g_scratch[dev].status = TB_OK;
}

int job_from_gemm(const tb_gemm_desc* d, Job* j) {
  if (!d) return TB_ERR_NULL_POINTER;
  if (d->struct_bytes != sizeof(tb_gemm_desc)) return TB_ERR_BAD_ARGUMENT;
  if (d->a_type != TB_F16 && d->a_type != TB_BF16 && d->a_type != TB_FP8_E4M3 && d->a_type != TB_FP8_E5M2 && d->a_type != TB_F32 &&
      d->a_type != TB_I8)
    return TB_ERR_BAD_DTYPE;
  const int dt = kernel_type(d->a_type, d->b_type);
  if (dt < 0) return TB_ERR_BAD_DTYPE;
  if ((d->a_scale == nullptr) != (d->b_scale == nullptr)) return TB_ERR_BAD_ARGUMENT;
  if (d->bias && d->bias_type != TB_F16 && d->bias_type != TB_BF16 && d->bias_type != TB_F32) return TB_ERR_BAD_DTYPE;
  j->dt = dt; j->c_type = d->c_type; j->bias_type = d->bias_type;
  j->M = d->m; j->N = d->n; j->K = d->k;
  j->A = d->a; j->B = d->b; j->C = d->c;
  j->a_sr = d->a_stride_m; j->a_sk = d->a_stride_k; j->b_sr = d->b_stride_n; j->b_sk = d->b_stride_k;
  j->c_sm = d->c_stride_m; j->c_sn = d->c_stride_n;
  j->sa = d->a_scale; j->sb = d->b_scale; j->bias = d->bias; j->bias_stride = d->bias_stride;
  j->bm = d->block_m; j->bn = d->block_n; j->bk = d->block_k; j->group_m = d->group_m; j->num_xcds = d->num_xcds;
  j->schedule = d->schedule; j->grid = d->grid; j->counters_per_xcd = d->counters_per_xcd;
  j->workspace = d->workspace; j->workspace_bytes = d->workspace_bytes; j->epoch = d->epoch; j->spin_limit = d->spin_limit;
  j->cu_mask = d->cu_mask; j->cu_mask_len = d->cu_mask_len; j->ws_mode = d->ws_mode;
  j->ws_local = d->ws_local_tiles_per_xcd; j->ws_global = d->ws_global_tiles;
  j->column_split = d->column_split;
  return TB_OK;
}

}  // namespace

extern "C" {

int tb_abi_version(void) { return TB_ABI_VERSION; }

int tb_tile_coords(int32_t tile, int32_t tiles_m, int32_t tiles_n, int32_t group_m, int32_t panel_n, int32_t* pm, int32_t* pn) {
  if (!pm || !pn) return TB_ERR_NULL_POINTER;
  if (tiles_m <= 0 || tiles_n <= 0 || group_m <= 0 || panel_n < 0 || tile < 0 || (int64_t)tile >= (int64_t)tiles_m * tiles_n) return TB_ERR_BAD_ARGUMENT;
  int m, n;
  tile_coords(tile, tiles_m, tiles_n, group_m, panel_n, m, n);
  *pm = m; *pn = n;
  return TB_OK;
}

int tb_ws_queue_tile(int32_t ws_mode, int32_t queue, int32_t idx, int32_t total_tiles, int32_t num_xcds,
                     int32_t counters_per_xcd, int32_t local_tiles_per_xcd, int32_t* count, int32_t* tile) {
  if (!count || !tile) return TB_ERR_NULL_POINTER;
  if (ws_mode < TB_WS_QUEUES || ws_mode > TB_WS_HIERARCHICAL || total_tiles <= 0 || num_xcds <= 0 || counters_per_xcd <= 0 ||
      queue < 0 || idx < 0 || local_tiles_per_xcd < 0)
    return TB_ERR_BAD_ARGUMENT;
  const int nq = ws_mode == TB_WS_QUEUES ? num_xcds * counters_per_xcd : ws_mode == TB_WS_GLOBAL_ATOMIC ? 1 : num_xcds + 1;
  if (queue >= nq) return TB_ERR_BAD_ARGUMENT;
  if (ws_mode == TB_WS_HIERARCHICAL && (int64_t)local_tiles_per_xcd * num_xcds > total_tiles) return TB_ERR_BAD_ARGUMENT;
  int first, cnt;
  ws_queue_range(ws_mode, queue, total_tiles, num_xcds, counters_per_xcd, local_tiles_per_xcd, first, cnt);
  *count = cnt;
  *tile = idx < cnt ? ws_queue_tile(ws_mode, first, idx, total_tiles, num_xcds) : -1;
  return TB_OK;
}

int tb_hierarchical_split(int64_t total_tiles, int32_t hw_cus, int32_t num_xcds, int32_t* local_tiles_per_xcd, int32_t* global_tiles) {
  if (!local_tiles_per_xcd || !global_tiles) return TB_ERR_NULL_POINTER;
  if (total_tiles <= 0 || total_tiles > INT32_MAX || hw_cus <= 0 || num_xcds <= 0) return TB_ERR_BAD_ARGUMENT;
  int64_t l, g;
  hierarchical_split(total_tiles, hw_cus, num_xcds, &l, &g);
  *local_tiles_per_xcd = (int32_t)l; *global_tiles = (int32_t)g;
  return TB_OK;
}

int tb_default_panel(int32_t grid, int32_t chunk, int32_t group_m) {
  if (grid <= 0 || chunk <= 0 || group_m <= 0) return TB_ERR_BAD_ARGUMENT;
  return default_panel_n(grid, chunk, group_m);
}

int tb_debug_option(const char* name, int value) {
  if (!name) return TB_ERR_NULL_POINTER;
  (void)hooks();
  std::lock_guard<std::mutex> lk(g_plan_mu);
  std::lock_guard<std::mutex> lk2(g_hooks_mu);
  struct { const char* n; int* p; } table[] = {
      {"waves", &g_hooks.waves}, {"no_mxlds", &g_hooks.no_mxlds}, {"no_cline", &g_hooks.no_cline},
      {"no_skinny", &g_hooks.no_skinny}, {"skinny", &g_hooks.skinny}, {"grid", &g_hooks.grid}, {"panel", &g_hooks.panel},
      {"no_column_split", &g_hooks.no_column_split}, {"force_column_split", &g_hooks.force_column_split}, {"quant_div64", &g_hooks.quant_div64}, {"lab", &g_hooks.lab},
      {"grp_sk_fix", &g_hooks.grp_sk_fix}};
  for (auto& t : table)
    if (std::strcmp(t.n, name) == 0) { *t.p = value; ++g_hooks_version; return TB_OK; }
  return TB_ERR_BAD_ARGUMENT;
}

int tb_workspace_layout(size_t* counters_offset, size_t* flags_offset) {
  if (!counters_offset || !flags_offset) return TB_ERR_NULL_POINTER;
  *counters_offset = WS_COUNTERS_OFF; *flags_offset = WS_FLAGS_OFF;
  return TB_OK;
}

const char* tb_status_string(int status) {
  switch (status) {
    case TB_OK: return "ok";
    case TB_ERR_NULL_POINTER: return "null pointer";
    case TB_ERR_BAD_SHAPE: return "Incompatible Dimensions";
    case TB_ERR_BAD_DTYPE: return "unsupported element type";
    case TB_ERR_BAD_LAYOUT: return "unsupported strides";
    case TB_ERR_BAD_TILE: return "no kernel variant for this tile";
    case TB_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
    case TB_ERR_BAD_SCHEDULE: return "invalid schedule or grid";
    case TB_ERR_LAUNCH: return "kernel launch failed";
    case TB_ERR_NO_DEVICE: return "no usable HIP device";
    case TB_ERR_BAD_ARGUMENT: return "bad argument";
  }
  return "unknown status";
}

int tb_device_info(int device, tb_hw* out) {
  if (!out) return TB_ERR_NULL_POINTER;
  if (device < 0) { default_hw(out); return TB_OK; }
  if (device >= MAX_DEVICES) return TB_ERR_BAD_ARGUMENT;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || device >= count) { (void)hipGetLastError(); return TB_ERR_NO_DEVICE; }
  std::call_once(g_hw_once[device], query_hw, device);
  if (g_hw_status[device] != TB_OK) return g_hw_status[device];
  *out = g_hw[device];
  return TB_OK;
}

int tb_list_tiles(int32_t a_type, int32_t* triples, int32_t cap) {
  auto infos = tile_infos(a_type);
  int n = 0;
  for (auto& t : infos) {
    if (!t.fast) continue;
    if (triples && n < cap) { triples[3 * n] = t.bm; triples[3 * n + 1] = t.bn; triples[3 * n + 2] = t.bk; }
    ++n;
  }
  return n;
}

int tb_select(const tb_problem* problem, const tb_hw* hw, tb_selection* out) {
  if (!problem || !out) return TB_ERR_NULL_POINTER;
  if (problem->m <= 0 || problem->n <= 0 || problem->k <= 0) return TB_ERR_BAD_SHAPE;
  tb_hw local;
  if (hw) local = *hw; else default_hw(&local);
  const int dt = kernel_type(problem->a_type, problem->b_type);
  if (dt < 0) return TB_ERR_BAD_DTYPE;
  auto infos = tile_infos(dt);
  if (infos.empty()) return TB_ERR_BAD_DTYPE;
  tb_problem pr = *problem;
  pr.a_type = pr.b_type = model_type(dt);
  return select_tile(pr, local, infos.data(), (int)infos.size(), out);
}

int tb_gemm(const tb_gemm_desc* desc, void* stream) {
  Job j;
  int st = job_from_gemm(desc, &j);
  if (st != TB_OK) return st;
  if (!j.A || !j.B || !j.C) return TB_ERR_NULL_POINTER;
  if (desc->column_split < -1 || desc->column_split > 0) return TB_ERR_BAD_ARGUMENT;
  return launch_columns(j, (hipStream_t)stream);
}

int tb_gemm_static_workspace(const tb_gemm_desc* desc, void* stream) {
  Job j;
  int st = job_from_gemm(desc, &j);
  if (st != TB_OK) return st;
  if (!j.A || !j.B || !j.C) return TB_ERR_NULL_POINTER;
  if (desc->column_split < -1 || desc->column_split > 0) return TB_ERR_BAD_ARGUMENT;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return TB_ERR_NO_DEVICE;
  std::call_once(g_scratch_once[dev], init_scratch, dev);
  ScratchState& sc = g_scratch[dev];
  if (sc.status != TB_OK) return sc.status;
  j.workspace = sc.ptr;
  j.workspace_bytes = SCRATCH_BYTES;   // (a launch that needs more is refused with TB_ERR_WORKSPACE)
  // The array keeps the last call's contents (it starts as zeros): the queue counters rearm themselves, and
  // Stream-K launches are told apart by the count the workspace keeps in its own control block -- so the
  // call records nothing that a replay of a captured graph would repeat wrongly.
  j.epoch = TB_EPOCH_ON_DEVICE;
  return launch_columns(j, (hipStream_t)stream);
}

int tb_static_workspace_status(int* status, int clear) {
  if (!status) return TB_ERR_NULL_POINTER;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return TB_ERR_NO_DEVICE;
  std::call_once(g_scratch_once[dev], init_scratch, dev);
  ScratchState& sc = g_scratch[dev];
  if (sc.status != TB_OK) return sc.status;
  // (the status word is control word CTL_STATUS of the array; the copy waits for the device's earlier work)
  uint32_t word = 0;
  uint8_t* at = (uint8_t*)sc.ptr + CTL_STATUS * 4;
  if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(&word, at, 4, hipMemcpyDeviceToHost) != hipSuccess) return TB_ERR_LAUNCH;
  if (clear && word != 0) {
    const uint32_t zero = 0;
    if (hipMemcpy(at, &zero, 4, hipMemcpyHostToDevice) != hipSuccess) return TB_ERR_LAUNCH;
  }
  *status = (int)word;
  return TB_OK;
}

int tb_gemm_launch_info(const tb_gemm_desc* desc, tb_launch_info* out) {
  if (!out) return TB_ERR_NULL_POINTER;
  Job j;
  int st = job_from_gemm(desc, &j);
  if (st != TB_OK) return st;
  tb_hw hw;
  const bool have_dev = current_hw(&hw) == TB_OK;
  if (!have_dev) default_hw(&hw);
  Plan plan;
  st = make_plan(j, hw, have_dev, &plan);
  if (st != TB_OK) return st;
  std::memset(out, 0, sizeof(*out));
  out->block_m = plan.v->bm; out->block_n = plan.v->bn; out->block_k = plan.v->bk;
  out->waves = plan.v->threads / 64; out->four_wave = plan.v->k_step_pairs ? 1 : 0;
  out->mode = plan.p.mode; out->grid = plan.grid; out->total_tiles = plan.p.total_tiles;
  out->sk_tiles = plan.p.mode == MODE_SK ? plan.p.sk_tiles : 0;
  out->sk_unit = plan.p.mode == MODE_SK ? std::max(1, plan.p.sk_unit) : 0;
  out->sk_ws = plan.p.sk_ws; out->skinny = plan.skinny ? 1 : 0;
  return TB_OK;
}

size_t tb_workspace_bytes(const tb_gemm_desc* desc) {
  Job j;
  if (job_from_gemm(desc, &j) != TB_OK) return 0;
  tb_hw hw;
  bool have_dev = current_hw(&hw) == TB_OK;
  if (!have_dev) default_hw(&hw);
  // alignment of the real pointers decides the kernel family; with null pointers assume aligned
  Plan plan;
  if (make_plan(j, hw, have_dev, &plan) != TB_OK) return 0;
  return plan.ws_need;
}

int tb_gemm_fp4(const tb_gemm_fp4_desc* d, void* stream) {
  if (!d) return TB_ERR_NULL_POINTER;
  if (d->struct_bytes != sizeof(tb_gemm_fp4_desc)) return TB_ERR_BAD_ARGUMENT;
  if (!d->a || !d->b || !d->c || !d->a_scales || !d->b_scales) return TB_ERR_NULL_POINTER;
  if (d->k <= 0 || d->k % 32) return TB_ERR_BAD_SHAPE;
  Job j;
  j.dt = TB_FP4_E2M1; j.c_type = d->c_type;
  j.M = d->m; j.N = d->n; j.K = d->k;
  j.A = d->a; j.B = d->b; j.C = d->c;
  j.a_sr = d->a_stride_m; j.a_sk = 1; j.b_sr = d->b_stride_n; j.b_sk = 1;
  j.c_sm = d->c_stride_m; j.c_sn = d->c_stride_n;
  j.mxa = d->a_scales; j.mxb = d->b_scales;
  j.mxa_sr = d->a_scales_stride_m; j.mxa_sk = d->a_scales_stride_k;
  j.mxb_sr = d->b_scales_stride_n; j.mxb_sk = d->b_scales_stride_k;
  j.bm = d->block_m; j.bn = d->block_n; j.bk = d->block_k; j.group_m = d->group_m; j.num_xcds = d->num_xcds;
  return launch(j, (hipStream_t)stream);
}

// the short FP8 tile the second launch of a grouped GEMM runs
constexpr int kGroupedSmallBM = 32, kGroupedSmallBN = 128, kGroupedSmallBK = 256;

// the job of the (first) launch; *two: a second launch with the short tile may follow
static int job_from_grouped(const tb_grouped_gemm_desc* d, Job* out, bool* two) {
  if (!d) return TB_ERR_NULL_POINTER;
  if (d->struct_bytes != sizeof(tb_grouped_gemm_desc)) return TB_ERR_BAD_ARGUMENT;
  if ((d->a_scale == nullptr) != (d->w_scale == nullptr)) return TB_ERR_BAD_ARGUMENT;
  if (d->num_groups <= 0) return TB_ERR_BAD_SHAPE;
  Job j;
  j.dt = TB_FP8_E4M3; j.c_type = d->c_type;
  j.M = d->m_total; j.N = d->n; j.K = d->k;
  j.A = d->a; j.B = d->w; j.C = d->c;
  j.a_sr = d->a_stride_m; j.a_sk = 1; j.b_sr = d->w_stride_n; j.b_sk = 1;
  j.c_sm = d->c_stride_m; j.c_sn = d->c_stride_n;
  j.sa = d->a_scale; j.sb = d->w_scale;
  j.bm = d->block_m; j.bn = d->block_n; j.bk = d->block_k; j.group_m = d->group_m; j.num_xcds = d->num_xcds;
  j.group_offsets = d->group_offsets; j.num_groups = d->num_groups;
  j.b_group_stride = d->w_stride_g; j.sb_group_stride = d->n;
  if ((d->w_stride_g * 1) % 16) return TB_ERR_BAD_LAYOUT;
  if (d->streamk < 0 || d->streamk > 1) return TB_ERR_BAD_ARGUMENT;
  if (d->streamk) {
    j.grp_sk = 1;
    j.workspace = d->workspace; j.workspace_bytes = d->workspace_bytes;
    j.epoch = d->epoch; j.spin_limit = d->spin_limit;
  }
  // Two launches unless switched off or a tile is forced: tall tiles for whole row blocks and long
  // remainders, then a short streaming tile for the experts whose last block holds few rows (the row
  // counts live on the device, so both tile tables are evaluated there; an empty second table costs
  // one empty launch).
  if (d->small_rows < -1) return TB_ERR_BAD_ARGUMENT;
  const int thr = d->small_rows > 0 ? d->small_rows : 64;
  *two = (d->small_rows > 0 || (d->small_rows == 0 && d->block_m == 0)) && d->k % kGroupedSmallBK == 0;
  if (*two) { j.grp_phase = 1; j.grp_thr = thr; j.grp_auto = d->small_rows == 0; }
  *out = j;
  return TB_OK;
}

size_t tb_grouped_workspace_bytes(const tb_grouped_gemm_desc* d) {
  Job j;
  bool two = false;
  if (job_from_grouped(d, &j, &two) != TB_OK || !j.grp_sk) return 0;
  tb_hw hw;
  bool have_dev = current_hw(&hw) == TB_OK;
  if (!have_dev) default_hw(&hw);
  Plan plan;
  if (make_plan(j, hw, have_dev, &plan) != TB_OK) return 0;
  return plan.ws_need;
}

int tb_streamk_tail_tiles(int32_t total_tiles, int32_t grid, int32_t k_units, int32_t unit_steps, int32_t fix_steps) {
  if (total_tiles < 0 || grid <= 0 || k_units <= 0 || unit_steps <= 0 || fix_steps < 0) return TB_ERR_BAD_ARGUMENT;
  return sk_tail_tiles(total_tiles, grid, k_units, unit_steps, fix_steps);
}

int tb_grouped_gemm_fp8(const tb_grouped_gemm_desc* d, void* stream) {
  if (!d) return TB_ERR_NULL_POINTER;
  if (d->struct_bytes != sizeof(tb_grouped_gemm_desc)) return TB_ERR_BAD_ARGUMENT;
  if (!d->a || !d->w || !d->c || !d->group_offsets) return TB_ERR_NULL_POINTER;
  Job j;
  bool two = false;
  int st = job_from_grouped(d, &j, &two);
  if (st != TB_OK) return st;
  if (!two) return launch(j, (hipStream_t)stream);
  tb_hw hw;
  st = current_hw(&hw);
  if (st != TB_OK) return st;
  Plan first, second;
  st = cached_plan(j, hw, &first);
  if (st != TB_OK) return st;
  if (first.p.grp_phase != 1) return run_plan(j, first, (hipStream_t)stream);
  Job j2 = j;
  j2.bm = kGroupedSmallBM; j2.bn = kGroupedSmallBN; j2.bk = kGroupedSmallBK;
  j2.grp_phase = 2; j2.grp_big = first.p.grp_big;
  j2.grp_sk = 0; j2.workspace = nullptr; j2.workspace_bytes = 0;
  st = cached_plan(j2, hw, &second);
  if (st != TB_OK) return st;
  first.p.grp_small_bm = second.p.grp_small_bm = second.v->bm;
  first.p.grp_other_tn = second.p.tiles_n; first.p.grp_other_grid = second.grid;
  second.p.grp_other_tn = first.p.tiles_n; second.p.grp_other_grid = first.grid;
  st = run_plan(j, first, (hipStream_t)stream);
  if (st != TB_OK) return st;
  return run_plan(j2, second, (hipStream_t)stream);
}

int tb_hadamard_mxfp4_quant(const tb_quant_desc* d, void* stream) {
  if (!d) return TB_ERR_NULL_POINTER;
  if (d->struct_bytes != sizeof(tb_quant_desc)) return TB_ERR_BAD_ARGUMENT;
  if (!d->x || !d->codes || !d->scales) return TB_ERR_NULL_POINTER;
  if (d->m <= 0 || d->n <= 0 || d->n % 32) return TB_ERR_BAD_SHAPE;
  if (d->x_type != TB_F16 && d->x_type != TB_BF16 && d->x_type != TB_F32) return TB_ERR_BAD_DTYPE;
  const int xb = d->x_type == TB_F32 ? 4 : 2;
  if (!aligned16(d->x) || (d->x_stride_m * xb) % 16 || ((uintptr_t)d->codes & 3) || d->codes_stride_m % 4) return TB_ERR_BAD_LAYOUT;
  QuantParams p;
  p.x = (const uint8_t*)d->x; p.codes = (uint8_t*)d->codes; p.scales = (uint8_t*)d->scales;
  p.m = d->m; p.n = d->n; p.x_stride = d->x_stride_m; p.codes_stride = d->codes_stride_m; p.scales_stride = d->scales_stride_m;
  hipError_t e = launch_quant(p, d->x_type, d->hadamard != 0, hooks().quant_div64 != 0, (hipStream_t)stream);
  if (e != hipSuccess) return TB_ERR_LAUNCH;
  return TB_OK;
}

}  // extern "C"
