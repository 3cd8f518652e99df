// INT8 tile GEMM kernels (v_mfma_i32_16x16x64_i8, exact int32 sums over the K range of a work item).
// K-major operands take the LDS-direct kernels, everything else the element-wise-gather kernel.
#include "gemm_variants.h"

namespace tb {

const Variant g_variants_i8[] = {
    make_variant_w4<W4Tile<DT_I8>>(),
    make_variant<Tile<DT_I8, 256, 256, 128, 2, 4, LAY_K, LAY_K, 1, true, 2>>(),
    make_variant<Tile<DT_I8, 128, 128, 128, 2, 2, LAY_K, LAY_K, 2, true, 2>>(),
    make_variant<Tile<DT_I8, 64, 64, 128, 2, 2, LAY_K, LAY_K, 4, true, 2>>(),
    make_variant<Tile<DT_I8, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, false, 2>>(),
};
const int g_num_variants_i8 = sizeof(g_variants_i8) / sizeof(Variant);

}  // namespace tb
