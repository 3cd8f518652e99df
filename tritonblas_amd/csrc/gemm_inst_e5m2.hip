// FP8 (OCP e5m2) tile GEMM kernels: the e4m3 kernels of gemm_inst_fp8.hip with the other format field in
// their MFMAs (the reference lists the type next to e4m3, include/tritonblas/utils.py:46).
#include "gemm_variants.h"

namespace tb {

const Variant g_variants_e5m2[] = {
    make_variant_w4<W4Tile<DT_E5M2>>(),
    make_variant<Tile<DT_E5M2, 256, 256, 128, 2, 4, LAY_K, LAY_K, 1, true, 2>>(),
    make_variant<Tile<DT_E5M2, 128, 128, 128, 2, 2, LAY_K, LAY_K, 2, true, 2>>(),
    make_variant<Tile<DT_E5M2, 64, 64, 128, 2, 2, LAY_K, LAY_K, 4, true, 2>>(),
    make_variant<Tile<DT_E5M2, 32, 128, 256, 1, 4, LAY_K, LAY_K, 1, true, 3>>(),
    make_variant<Tile<DT_E5M2, 64, 64, 128, 2, 2, LAY_K, LAY_K, 3, true, 3>>(),
    make_variant<Tile<DT_E5M2, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, true, 4>>(),
    make_variant<Tile<DT_E5M2, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, false, 2>>(),
};
const int g_num_variants_e5m2 = sizeof(g_variants_e5m2) / sizeof(Variant);

}  // namespace tb
