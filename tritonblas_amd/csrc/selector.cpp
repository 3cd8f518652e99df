// Analytical tile selector for the gfx950 kernel family: scores every built tile variant with a
// small roofline-style model (MFMA issue time, LDS read time, L2->LDS fill time, wave quantisation
// over the CUs, HBM time) and derives the launch parameters that go with the winner (GROUP_M, XCD
// remap, Stream-K grid, work-stealing slots).
#include <algorithm>
#include <cmath>
#include <cstring>
#include "selector.h"

namespace tb {

static int type_bits(int t) {
  switch (t) {
    case TB_F16: case TB_BF16: return 16;
    case TB_FP8_E4M3: return 8;
    case TB_FP4_E2M1: return 4;
    case TB_F32: return 32;
  }
  return 0;
}

// dense MFMA flops per clock per CU
static double mfma_flops_per_clk(int t) {
  switch (t) {
    case TB_F16: case TB_BF16: return 4096.0;
    case TB_FP8_E4M3: return 8192.0;
    case TB_FP4_E2M1: return 16384.0;
  }
  return 1024.0;
}

void default_hw(tb_hw* hw) {
  std::memset(hw, 0, sizeof(*hw));
  hw->n_cu = 256; hw->num_xcd = 8; hw->cu_per_xcd = 32; hw->lds_bytes = 163840; hw->l2_bytes = 4 << 20;
  hw->clock_khz = 2400000; hw->mem_clock_khz = 2000000; hw->wave_size = 64; hw->hbm_gbps = 8000.0;
  std::strncpy(hw->arch, "gfx950", sizeof(hw->arch) - 1);
}

int ws_counters_per_xcd(int64_t total_tiles) {
  if (total_tiles <= 512) return 8;
  if (total_tiles <= 1536) return 4;
  if (total_tiles <= 2048) return 2;
  return 1;
}

static int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Workgroups of one variant that fit a CU (LDS and wave slots), capped by what the kernel was built for.
int variant_occupancy(const TileInfo& v, const tb_hw& hw) {
  int by_lds = std::max(1, hw.lds_bytes / std::max(1, v.lds_bytes));
  int by_waves = std::max(1, (8 * 4) / (v.threads / 64));
  return std::max(1, std::min({by_lds, by_waves, v.minb}));
}

// Measured behaviour of the built kernels on MI355X that the model is anchored to:
//   * MFMA-side efficiency of the K loop with operands already in LDS (fraction of the matrix pipe):
//     256x256 tiles ~0.47, 128x128 ~0.64, 64x64 ~0.55, the skinny 32x128 tile ~0.30;
//   * L2 -> LDS fill rate per CU: ~16 B/clk with one workgroup per CU, ~30 B/clk with two or more
//     (the vector L1 keeps a bounded number of lines in flight, so the rate is latency-bound).
static double mfma_side_efficiency(const TileInfo& v) {
  const int area = v.bm * v.bn;
  if (area >= 256 * 256) return 0.47;
  if (area >= 128 * 128) return 0.64;
  if (area >= 64 * 64) return 0.55;
  return 0.30;
}

static double score(const tb_problem& pr, const tb_hw& hw, const TileInfo& v, bool streamk, double* comp_us,
                    double* mem_us) {
  const double clk = hw.clock_khz * 1e3;
  const int bits = type_bits(pr.a_type);
  const double esz = bits / 8.0;
  const int64_t tiles_m = cdiv(pr.m, v.bm), tiles_n = cdiv(pr.n, v.bn);
  const int64_t tiles = tiles_m * tiles_n + (pr.num_groups > 0 ? (int64_t)pr.num_groups * tiles_n / 2 : 0);
  const int64_t k_iters = cdiv(pr.k, v.bk);
  const int occ = variant_occupancy(v, hw);
  const double bkb = v.bk * esz;

  // per K step of one workgroup, in CU cycles (MFMA pipe and fill path are shared by the CU)
  const double t_mfma = 2.0 * v.bm * v.bn * v.bk / mfma_flops_per_clk(pr.a_type) / mfma_side_efficiency(v);
  const double t_fill = (v.bm + v.bn) * bkb / (occ >= 2 ? 30.0 : 16.0);
  const double t_iter = std::max(t_mfma, t_fill) + 60.0;
  const double c_bytes = type_bits(pr.c_type) / 8.0;
  const double t_epi = 2500.0 + v.bm * v.bn * c_bytes / 32.0;

  double cycles;
  if (streamk) {
    // K iterations spread evenly over every resident workgroup slot; one partial-tile fixup each
    const double slots = (double)hw.n_cu * occ;
    const double iters_per_cu = std::ceil((double)tiles * k_iters / slots) * occ;
    cycles = iters_per_cu * t_iter + t_epi * std::max(1.0, (double)tiles / slots) + 6000.0;
  } else {
    const double rounds = std::ceil((double)tiles / (double)hw.n_cu);  // tiles one CU works through
    cycles = rounds * (k_iters * t_iter + t_epi / occ);
    // a partly filled last round leaves CUs idle; small grids cannot use the L2-hit fill rate either
    if (tiles < hw.n_cu) cycles = k_iters * t_iter + t_epi;
  }
  *comp_us = cycles / clk * 1e6;

  // HBM: every operand once, plus re-reads when a band of tiles does not stay in L2/MALL
  const double a_bytes = (double)pr.m * pr.k * esz, b_bytes = (double)pr.n * pr.k * esz * std::max(1, pr.num_groups);
  const double c_out = (double)pr.m * pr.n * c_bytes;
  // few workgroups cannot pull the full HBM rate: ~45 GB/s per busy CU
  const double busy_cus = std::min<double>(hw.n_cu, streamk ? hw.n_cu : (double)tiles);
  const double hbm = std::min(hw.hbm_gbps * 0.65, busy_cus * 45.0);
  *mem_us = (a_bytes + b_bytes + c_out) / (hbm * 1e9) * 1e6;
  return std::max(*comp_us, *mem_us) + 3.0;
}

int select_tile(const tb_problem& pr, const tb_hw& hw, const TileInfo* tiles, int ntiles, tb_selection* out) {
  int best = -1;
  double best_t = 0, best_c = 0, best_m = 0;
  for (int i = 0; i < ntiles; ++i) {
    const TileInfo& v = tiles[i];
    if (!v.fast) continue;  // the gather kernels are a fallback, never a choice of the model
    if (v.lds_bytes > hw.lds_bytes) continue;
    // decode-like problems (a handful of rows): tiles taller than twice the row count only add
    // LDS traffic and idle MFMA rows when a shorter tile exists
    bool shorter_exists = false;
    for (int q = 0; q < ntiles; ++q) shorter_exists |= tiles[q].fast && tiles[q].bm < v.bm && tiles[q].bm >= pr.m;
    if (shorter_exists && pr.num_groups == 0) continue;
    if (pr.num_groups > 0) {
      // grouped: the row counts live on the device; size the tile for the average group so that the
      // ragged last row block of each group wastes little
      const int64_t avg = std::max<int64_t>(1, pr.m / pr.num_groups);
      const int want = avg >= 192 ? 256 : (avg >= 96 ? 128 : 64);
      if (v.bm != want || v.bn != want) continue;
    }
    double c, m;
    double t = score(pr, hw, v, pr.streamk != 0, &c, &m);
    // prefer the larger tile on ties (less L2 traffic than the model resolves)
    if (best < 0 || t < best_t * 0.995 || (t <= best_t * 1.005 && (int64_t)v.bm * v.bn > (int64_t)tiles[best].bm * tiles[best].bn)) {
      best = i; best_t = t; best_c = c; best_m = m;
    }
  }
  if (best < 0) return TB_ERR_BAD_TILE;
  const TileInfo& v = tiles[best];
  std::memset(out, 0, sizeof(*out));
  out->block_m = v.bm; out->block_n = v.bn; out->block_k = v.bk;
  const int64_t tiles_m = cdiv(pr.m, v.bm), tiles_n = cdiv(pr.n, v.bn);
  const int64_t total = tiles_m * tiles_n;
  out->group_m = (int)std::min<int64_t>(8, tiles_m);
  out->num_xcds = hw.num_xcd;
  out->occupancy = variant_occupancy(v, hw);
  out->num_stages = v.stages;
  out->lds_bytes = v.lds_bytes;
  out->counters_per_xcd = ws_counters_per_xcd(total);
  // Stream-K grid: every resident workgroup slot, but never more workgroups than K iterations to share
  const int64_t k_iters = cdiv(pr.k, v.bk);
  int64_t grid = (int64_t)hw.n_cu * out->occupancy;
  grid = std::min(grid, total * k_iters);
  if (total % grid == 0 && total >= grid) grid = std::min<int64_t>(grid, total);
  out->sk_grid = (int)std::max<int64_t>(1, grid);
  out->est_compute_us = best_c; out->est_memory_us = best_m; out->est_total_us = best_t;
  return TB_OK;
}

}  // namespace tb
