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
    case TB_FP8_E4M3: case TB_FP8_E5M2: case TB_I8: return 8;
    case TB_FP4_E2M1: return 4;
    case TB_F32: return 32;
  }
  return 0;
}

// dense MFMA flops per clock per CU
static double mfma_flops_per_clk(int t) {
  switch (t) {
    case TB_F16: case TB_BF16: return 4096.0;
    case TB_FP8_E4M3: case TB_FP8_E5M2: case TB_I8: return 8192.0;
    case TB_FP4_E2M1: return 16384.0;
    case TB_F32: return 256.0;
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

// Reference origami.py:288-311: up to 4 tiles per CU everything stays XCD-local; above that the local
// share falls by 5 % per extra tile per CU, down to one half.  The local queues never get more than
// divides evenly (the reference's formula hands out one tile per XCD even when there are fewer tiles
// than XCDs).
void hierarchical_split(int64_t total_tiles, int hw_cus, int num_xcds, int64_t* local_per_xcd, int64_t* global_tiles) {
  const double tiles_per_cu = (double)total_tiles / std::max(hw_cus, 1);
  const double local_frac = std::max(0.5, 1.0 - std::max(0.0, tiles_per_cu - 4.0) * 0.05);
  int64_t local = std::max<int64_t>((int64_t)((double)total_tiles * local_frac) / num_xcds, 1);
  local = std::min(local, total_tiles / num_xcds);
  *local_per_xcd = local;
  *global_tiles = total_tiles - local * num_xcds;
}

static int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Workgroups of one variant that fit a CU (LDS and wave slots), capped by what the kernel was built for.
int variant_occupancy(const TileInfo& v, const tb_hw& hw) {
  int by_lds = std::max(1, hw.lds_bytes / std::max(1, v.lds_bytes));
  int by_waves = std::max(1, (8 * 4) / (v.threads / 64));
  return std::max(1, std::min({by_lds, by_waves, v.minb}));
}

// Measured behaviour of the built kernels on MI355X that the model is anchored to (8192-class
// problems for the saturated rates, 128..2048-row problems for the latency floor):
//   * a CU that is kept busy by `occ` resident workgroups finishes one K step of one tile every
//     ideal_step / eff: eff = fraction of the MFMA peak the kernel family sustains for that tile area;
//   * a workgroup cannot turn a K step around faster than ~0.3 us (barrier + L2 round trip) plus the
//     time its own copy takes at the ~100 GB/s one workgroup pulls (0.46 us for a 16 KB step, 0.65 us
//     for 40 KB): small problems want enough tiles to put several workgroups on every CU, and
//     long-K problems with few rows want the deep 32x128x256 tile;
//   * per tile: epilogue + first-copy latency, ~12 us for 256x256 (8 us on the 4-wave kernel), ~4 us for 128x128, ~3 us below.
// w4: the hand-scheduled 4-wave kernel runs the 256x256 tile (K an even number of K steps, at least four); its
// figures are from rounds of 256 tiles at K = 4096 and 8192 (FP8 46.5 and 85.7 us per round, bf16 89 and 178 us,
// MXFP4 8192x8192x16384 in 0.40-0.43 ms) with 8 us per tile.
static double family_efficiency(int dt, const TileInfo& v, bool w4) {
  const int area = v.bm * v.bn;
  const int cls = (v.bm < 64 || v.bn < 64) ? 3 : (area >= 256 * 256 ? 0 : (area >= 128 * 128 ? 1 : 2));
  if (w4 && cls == 0) {
    if (dt == TB_FP8_E4M3 || dt == TB_FP8_E5M2 || dt == TB_I8) return 0.705;
    if (dt == TB_FP4_E2M1) return 0.56;
    if (dt == TB_F16 || dt == TB_BF16) return 0.655;
  }
  static const double f8[4] = {0.61, 0.46, 0.29, 0.15};     // (128x128: 8192x28672x8192 in 1.72-1.77 ms, 8192^3 in 0.48 ms)
  static const double h16[4] = {0.59, 0.465, 0.22, 0.12};  // (128x128: 8192^3 bf16 in 0.97 ms)
  static const double f4[4] = {0.50, 0.36, 0.22, 0.10};     // (256x256: the 4-wave kernel, 8192x8192x16384 in 0.43-0.47 ms)
  static const double f32[4] = {0.80, 0.75, 0.60, 0.30};   // the fp32 matrix pipe is slow enough to hide everything else
  if (dt == TB_FP8_E4M3 || dt == TB_FP8_E5M2 || dt == TB_I8) return f8[cls];
  if (dt == TB_FP4_E2M1) return f4[cls];
  if (dt == TB_F32) return f32[cls];
  return h16[cls];
}

// Stream-K launch grid for `total` tiles of `k_iters` K steps on `slots` co-resident workgroups of `n_cu` CUs.
//   * at least one whole tile per CU, but fewer tiles than slots: one workgroup per tile, nothing is
//     split -- every CU is busy, and cutting tiles only to raise the occupancy costs more in partial-tile
//     traffic than it gains (measured: 64x28672x8192 fp8, 448 tiles of 64x64: 38 us whole, 60 us in halves);
//   * fewer tiles than CUs: every tile is cut into the same number s of K segments (grid = total * s).
//     s is a power of two (segment counts that do not divide the K steps evenly were up to 2x slower:
//     32x4096x14336 bf16, 112 steps: s = 4 and 8 28 us, s = 5..7 31..53 us), at most what fits the slots,
//     never leaving fewer than 8 K steps per segment, and the one that minimises
//     steps_per_segment * step_us + (s - 1) * fix_us -- the owner adds the other segments' partial tiles
//     one after the other;
//   * tiles >= slots: every slot takes part: whole tiles first, the last total % slots tiles are shared --
//     unless another round of whole tiles is expected to be as fast (large tiles have expensive partial
//     tiles: 2048x14336x4096 bf16, 448 tiles of 256x256 on 256 slots: 209 us in two rounds, 253 us with a
//     shared tail); the return value `total` means "whole tiles only".
// A last round that does not fill the CUs is cheaper than a full one for the 256x256 tiles (one workgroup per CU):
// the busy CUs run at a higher clock and share the L2s and the fabric with fewer others.  Measured, FP8 and bf16,
// K = 4096 and 8192, as a fraction of a full round: 0.66-0.69 with 6 % of the CUs busy, 0.84-0.91 with a quarter,
// 0.87-0.93 with half or three quarters.  f: the busy fraction.
static double partial_round_factor(double f) {
  if (f <= 0.0 || f >= 1.0) return 1.0;
  return f < 0.25 ? 0.65 + f : (f < 0.75 ? 0.9 : 0.9 + 0.4 * (f - 0.75));
}
static const double kSharedTailFactor = 4.0;
// What the exchange of partial tiles costs the workgroup that finishes a tile cut into `segments` pieces, when
// `partials` partial tiles are exchanged at about the same time.  xchg_us = 0 (the 8-wave kernels): fix_us per extra
// piece, one after the other, times `crowd` when a whole grid shares a tail.  xchg_us > 0 (the 4-wave 256x256 kernels,
// whose pieces exchange 256 KB each): the exchange is bound by what all of them move together -- 128 tiles cut in two
// 30 us, 64 tiles cut in four 43 us, a tail of 280 tiles shared by 256 workgroups 60 us: 0.23 us per partial tile,
// about 1.1 TB/s -- and never faster than one workgroup reads its partners' tiles (fix_us each).
static double exchange_us(double segments, double partials, double fix_us, double xchg_us, double crowd) {
  if (segments <= 1.0) return 0.0;
  if (xchg_us > 0.0) return std::max((segments - 1.0) * fix_us, partials * xchg_us);
  return (segments - 1.0) * fix_us * crowd;
}
int streamk_grid(int64_t total, int64_t k_iters, int slots, int n_cu, double step_us, double fix_us, double xchg_us) {
  if (total <= 0 || slots <= 0) return 1;
  if (total >= slots) {
    const int64_t tail = total % slots;
    if (tail == 0) return slots;
    // (a tail shared by the whole grid costs about four times the per-segment figure that the split of
    // a few tiles shows: 2048x28672x8192 FP8, 128 tiles of 256x256 shared by 256 workgroups, ~100 us on
    // top of their K steps; 1024x28672x8192, 192 shared tiles, the same)
    const double segments = std::ceil((double)slots / tail);
    const double shared = std::ceil((double)tail * k_iters / slots) * step_us +
                          exchange_us(segments, (double)(slots - tail), fix_us, xchg_us, kSharedTailFactor);
    const double whole = (double)k_iters * step_us * (xchg_us > 0.0 ? partial_round_factor((double)tail / slots) : 1.0);
    return shared < whole ? slots : (int)std::min<int64_t>(total, INT32_MAX);
  }
  if (total >= n_cu) return (int)total;
  const int64_t smax = std::max<int64_t>(1, slots / total);
  int64_t best_s = 1;
  double best = 0;
  for (int64_t s2 = 1; s2 <= smax && (s2 == 1 || k_iters / s2 >= 8); s2 *= 2) {
    // workgroups per CU grow with the split; beyond one per CU they share its matrix pipe
    const double share = std::max(1.0, (double)(total * s2) / n_cu);
    const double cost = std::ceil((double)k_iters / s2) * step_us * std::sqrt(share) +
                        exchange_us((double)s2, (double)(total * (s2 - 1)), fix_us, xchg_us, 1.0);
    if (s2 == 1 || cost < best) { best = cost; best_s = s2; }
  }
  return (int)(total * best_s);
}

static double score(const tb_problem& pr, const tb_hw& hw, const TileInfo& v, bool streamk, double* comp_us,
                    double* mem_us, int* sk_grid_out = nullptr) {
  const double clk = hw.clock_khz * 1e3;
  const int bits = type_bits(pr.a_type);
  const double esz = bits / 8.0;
  const int64_t tiles_m = cdiv(pr.m, v.bm), tiles_n = cdiv(pr.n, v.bn);
  const int64_t tiles = tiles_m * tiles_n + (pr.num_groups > 0 ? (int64_t)pr.num_groups * tiles_n / 2 : 0);
  const int64_t k_iters = cdiv(pr.k, v.bk);
  const int occ = variant_occupancy(v, hw);
  const int area = v.bm * v.bn;

  const double ideal_step_us = 2.0 * v.bm * v.bn * v.bk / mfma_flops_per_clk(pr.a_type) / clk * 1e6;
  const bool w4 = v.threads == 256 && area >= 256 * 256 && k_iters >= 4 && k_iters % 2 == 0;
  const double t_thru = ideal_step_us / family_efficiency(pr.a_type, v, w4);   // CU time per tile K step, saturated
  double t_lat = 0.30 + (v.bm + v.bn) * (v.bk * esz) / 1.0e5;                // floor per K step of one workgroup: round trip + its own copy at ~100 GB/s
  // the 64x64 tile of the 8- and 16-bit float types runs with four (three) copy stages while no more
  // than two (three) tiles per CU exist, which hides that much more of the round trip (measured x0.67 / x0.85)
  if (v.bm == 64 && v.bn == 64 && pr.num_groups == 0 &&
      (pr.a_type == TB_F16 || pr.a_type == TB_BF16 || pr.a_type == TB_FP8_E4M3 || pr.a_type == TB_FP8_E5M2)) {
    const int64_t whole = cdiv(pr.m, v.bm) * cdiv(pr.n, v.bn);
    if (whole <= 2 * (int64_t)hw.n_cu) t_lat *= 0.67;
    else if (whole <= 3 * (int64_t)hw.n_cu) t_lat *= 0.85;
  }
  // the FP8 128x128 tile runs with four copy stages while every tile has a CU of its own
  if (v.bm == 128 && v.bn == 128 && pr.num_groups == 0 && pr.a_type == TB_FP8_E4M3 &&
      cdiv(pr.m, v.bm) * cdiv(pr.n, v.bn) <= (int64_t)hw.n_cu)
    t_lat *= 0.67;
  const double t_tile = area >= 256 * 256 ? (w4 ? 8.0 : 12.0) : (area >= 128 * 128 ? 4.0 : 3.0);
  auto last_round = [&](int64_t n_tiles, int64_t per_round) {
    const int64_t r = n_tiles % per_round;
    if (r == 0 || area < 256 * 256) return 1.0;
    return partial_round_factor((double)r / per_round);
  };

  double us;
  if (streamk) {
    // one extra K segment of a tile costs its partial tile written through, polled for and added by the
    // owner, one after the other: ~1.5 us + the fp32 tile at ~10 GB/s (fitted on segment-count sweeps:
    // 32x128 tiles ~3 us, 128x128 tiles ~8 us, 256x256 tiles ~30 us per extra segment)
    // The 4-wave 256x256 kernels (256 threads) exchange partial tiles straight from the accumulators with 16 loads in
    // flight per lane: 4.5 us per partner for one workgroup alone, and 0.23 us per partial tile of the whole launch
    // (see exchange_us).
    const bool big4 = w4 && k_iters % 4 == 0;   // (the 4-wave Stream-K kernel cuts K at multiples of four steps)
    const double fix_us = big4 ? 4.5 : 1.5 + area * 4.0 / 10e3;
    const double xchg_us = big4 ? 0.23 : 0.0;
    const int slots = hw.n_cu * occ;
    const int grid = streamk_grid(tiles, k_iters, slots, hw.n_cu, std::max(t_thru, t_lat), fix_us, xchg_us);
    if (sk_grid_out) *sk_grid_out = grid;
    const int launched = (int)std::min<int64_t>(grid, slots);     // (grid == tiles > slots: whole tiles, resident grid loops)
    const double w = (double)cdiv(launched, hw.n_cu);             // workgroups sharing the busiest CU
    const double t_step = std::max(w * t_thru, t_lat);
    if (grid >= tiles && tiles > slots) {
      us = ((double)(cdiv(tiles, slots) - 1) + last_round(tiles, slots)) * (k_iters * t_step + t_tile);
    } else {
      const int64_t dp_rounds = tiles / grid, tail = tiles % grid;
      us = (double)dp_rounds * (k_iters * t_step + t_tile);
      if (tail > 0) {
        const double iters = std::ceil((double)tail * k_iters / grid);
        const double segments = std::ceil((double)grid / tail);
        // (tiles < grid: every tile is cut into `segments` pieces; otherwise a tail shared by the whole grid)
        const double partials = dp_rounds > 0 ? (double)(grid - tail) : (double)tail * (segments - 1.0);
        us += iters * t_step + exchange_us(segments, partials, fix_us, xchg_us, dp_rounds > 0 ? kSharedTailFactor : 1.0) + t_tile;
      }
    }
  } else {
    // the busiest CU works through c tiles, occ at a time
    const int64_t c = cdiv(tiles, hw.n_cu);
    const int64_t full = c / occ, rem = c % occ;
    us = (double)full * (k_iters * std::max(occ * t_thru, t_lat) + t_tile);
    if (rem) us += k_iters * std::max((double)rem * t_thru, t_lat) + t_tile;
    if (occ == 1 && c > 1) us -= (1.0 - last_round(tiles, hw.n_cu)) * (k_iters * std::max(t_thru, t_lat) + t_tile);
  }
  *comp_us = us;

  // HBM: every operand once
  const double c_bytes = type_bits(pr.c_type) / 8.0;
  const double a_bytes = (double)pr.m * pr.k * esz, b_bytes = (double)pr.n * pr.k * esz * std::max(1, pr.num_groups);
  const double c_out = (double)pr.m * pr.n * c_bytes;
  // few workgroups cannot pull the full HBM rate: ~45 GB/s per busy CU
  const double busy_cus = std::min<double>(hw.n_cu, streamk ? hw.n_cu : (double)tiles);
  const double hbm = std::min(hw.hbm_gbps * 0.65, busy_cus * 45.0);
  *mem_us = (a_bytes + b_bytes + c_out) / (hbm * 1e9) * 1e6;
  return std::max(*comp_us, *mem_us) + 3.0;
}

int streamk_grid_for(const tb_problem& pr, const tb_hw& hw, const TileInfo& v) {
  double c, m;
  int grid = 1;
  score(pr, hw, v, true, &c, &m, &grid);
  return grid;
}

double estimate_tile_us(const tb_problem& pr, const tb_hw& hw, const TileInfo& v, bool streamk) {
  double c, m;
  return score(pr, hw, v, streamk, &c, &m);
}

// The streaming kernel for a handful of rows: every workgroup owns 64 columns of the weight, reads them
// once from HBM (measured over the whole grid: ~4.6 TB/s with 8-bit operands, ~3.4 TB/s with 16-bit
// ones) and re-reads all of A from L2 (~17 TB/s over the grid); ~13 us of launch, split-K reduction and
// store on top.
double estimate_streaming_us(const tb_problem& pr, const tb_hw& hw) {
  const double esz = type_bits(pr.a_type) / 8.0;
  const double b_bytes = (double)pr.n * pr.k * esz;
  const double a_reread = std::ceil(pr.n / 64.0) * (double)pr.m * pr.k * esz;
  const double hbm = hw.hbm_gbps * (esz > 1.0 ? 0.425 : 0.575) * 1e3, l2 = hw.hbm_gbps * 2.125 * 1e3;   // bytes per us
  return 13.0 + b_bytes / hbm + a_reread / l2;
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
  out->sk_grid = streamk_grid_for(pr, hw, v);
  out->est_compute_us = best_c; out->est_memory_us = best_m; out->est_total_us = best_t;
  return TB_OK;
}

}  // namespace tb
