// fp32 tile GEMM kernels (v_mfma_f32_16x16x4_f32: full fp32 products and sums; this target has no
// reduced-precision fp32 matrix mode).  K-contiguous operands take the LDS-direct kernels; every
// other layout goes through the element-wise-gather kernel.
#include "gemm_variants.h"

namespace tb {

const Variant g_variants_f32[] = {
    make_variant<Tile<DT_F32, 256, 256, 128, 2, 4, LAY_K, LAY_K, 1, true, 2>>(),
    make_variant<Tile<DT_F32, 128, 128, 128, 2, 2, LAY_K, LAY_K, 2, true, 2>>(),
    make_variant<Tile<DT_F32, 64, 64, 128, 2, 2, LAY_K, LAY_K, 4, true, 2>>(),
    make_variant<Tile<DT_F32, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, false, 2>>(),
};
const int g_num_variants_f32 = sizeof(g_variants_f32) / sizeof(Variant);

}  // namespace tb
