// FP8 (OCP e4m3) tile GEMM kernels.  The fast kernels take K-major operands; everything else goes
// through the element-wise-gather kernel.
#include "gemm_variants.h"

namespace tb {

const Variant g_variants_fp8[] = {
    // hand-scheduled 4-wave kernel: taken when K is a multiple of two K steps and no Stream-K tail is asked for
    make_variant_w4<W4Tile<DT_FP8>>(),
    make_variant<Tile<DT_FP8, 256, 256, 128, 2, 4, LAY_K, LAY_K, 1, true, 2>>(),
    make_variant<Tile<DT_FP8, 128, 128, 128, 2, 2, LAY_K, LAY_K, 2, true, 2>>(),
    make_variant<Tile<DT_FP8, 64, 64, 128, 2, 2, LAY_K, LAY_K, 4, true, 2>>(),
    make_variant<Tile<DT_FP8, 32, 128, 256, 1, 4, LAY_K, LAY_K, 1, true, 3>>(),
    // deeper copy pipelines of the small tile for problems with few tiles per CU (each K step then
    // waits less for its copy; fewer workgroups fit a CU)
    // (the same for the 128x128 tile while every tile has a CU of its own: 128 KB of stages, one workgroup per CU;
    // 512x8192x8192 48 -> 39 us, 128x28672x8192 51 -> 42 us.  The 16-bit kernels lose with it: 80 -> 92 us.)
    make_variant<Tile<DT_FP8, 128, 128, 128, 2, 2, LAY_K, LAY_K, 1, true, 4>>(),
    make_variant<Tile<DT_FP8, 64, 64, 128, 2, 2, LAY_K, LAY_K, 3, true, 3>>(),
    make_variant<Tile<DT_FP8, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, true, 4>>(),
    make_variant<Tile<DT_FP8, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, false, 2>>(),
};
const int g_num_variants_fp8 = sizeof(g_variants_fp8) / sizeof(Variant);

}  // namespace tb
