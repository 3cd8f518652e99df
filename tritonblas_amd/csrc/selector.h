// Host-only: analytical tile selector.
#pragma once
#include <stdint.h>
#include "../../include/tritonblas_amd.h"

namespace tb {

struct TileInfo {
  int dt, bm, bn, bk, threads, lds_bytes, minb, fast, stages;
};

void default_hw(tb_hw* hw);
int streamk_grid(int64_t total_tiles, int64_t k_iters, int slots, int n_cu, double step_us, double fix_us, double xchg_us = 0.0);
// the Stream-K grid the model picks for one tile variant on a problem
int streamk_grid_for(const tb_problem& pr, const tb_hw& hw, const TileInfo& v);
int ws_counters_per_xcd(int64_t total_tiles);
// (tiles per XCD-local queue, tiles in the shared pool) of the hierarchical work-stealing mode
void hierarchical_split(int64_t total_tiles, int hw_cus, int num_xcds, int64_t* local_per_xcd, int64_t* global_tiles);
int variant_occupancy(const TileInfo& v, const tb_hw& hw);
int select_tile(const tb_problem& pr, const tb_hw& hw, const TileInfo* tiles, int ntiles, tb_selection* out);
// model time (us) of one tile variant on a problem, and of the streaming small-M kernel
double estimate_tile_us(const tb_problem& pr, const tb_hw& hw, const TileInfo& v, bool streamk);
double estimate_streaming_us(const tb_problem& pr, const tb_hw& hw);

}  // namespace tb
