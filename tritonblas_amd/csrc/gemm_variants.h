// Host-visible registry of the built GEMM kernel variants.
#pragma once
#include <stdint.h>
#include "gemm_device.h"

namespace tb {

struct Variant {
  int dt, bm, bn, bk;     // element type and tile in elements
  int alay, blay;         // operand loaders (LAY_K / LAY_M)
  int wm, wn, threads, lds_bytes, minb;
  int fast, stages;       // fast: vector/LDS-direct loaders (alignment + K multiple required)
  const void* kernel;     // __global__ void (*)(const GemmParams), whole-tile schedules
  const void* kernel_sk;  // same tile with the Stream-K tail (null: this variant has none)
  int k_step_pairs;       // 1: hand-scheduled 4-wave kernel -- K must be an even number of K steps, at least four; with a
                          // Stream-K tail a multiple of four (the K ranges of its pieces are cut at multiples of four steps)
};

template <class T>
constexpr Variant make_variant() {
  return Variant{T::DT, T::BM, T::BN, T::BK, T::ALAY, T::BLAY, T::WM, T::WN, T::THREADS, T::LDS_ALLOC, T::MINB,
                 T::FAST ? 1 : 0, T::STAGES, (const void*)&gemm_kernel<T, false>, (const void*)&gemm_kernel<T, true>, 0};
}

// The hand-scheduled 4-wave kernels of gemm_w4.h (256x256 tile, 128-byte K steps) are compiled in a
// translation unit of their own (gemm_inst_w4.hip), which hands out their addresses.
const void* w4_kernel(int dt);
const void* w4_kernel_sk(int dt);
template <int DT>
using W4Tile = Tile<DT, 256, 256, 128, 2, 2, LAY_K, LAY_K, 1, true, 2>;
// LDS of these kernels: two 64 KB stages, 16 KB of FP4 scale buffers, 1 KB per wave of epilogue scales,
// the schedule's broadcast word
constexpr int W4_EPS_OFFSET = 131072 + 16384;
constexpr int W4_LDS_BYTES = W4_EPS_OFFSET + 4096 + 16;
template <class T>
Variant make_variant_w4() {
  return Variant{T::DT, T::BM, T::BN, T::BK, T::ALAY, T::BLAY, T::WM, T::WN, T::THREADS, W4_LDS_BYTES, 1,
                 1, T::STAGES, w4_kernel(T::DT), w4_kernel_sk(T::DT), 1};
}

// defined one per translation unit
extern const Variant g_variants_f16[];
extern const int g_num_variants_f16;
extern const Variant g_variants_bf16[];
extern const int g_num_variants_bf16;
extern const Variant g_variants_fp8[];
extern const int g_num_variants_fp8;
extern const Variant g_variants_e5m2[];
extern const int g_num_variants_e5m2;
extern const Variant g_variants_e4e5[];
extern const int g_num_variants_e4e5;
extern const Variant g_variants_e5e4[];
extern const int g_num_variants_e5e4;
extern const Variant g_variants_fp4[];
extern const int g_num_variants_fp4;
extern const Variant g_variants_f32[];
extern const int g_num_variants_f32;
extern const Variant g_variants_i8[];
extern const int g_num_variants_i8;

}  // namespace tb
