// FP8 tile GEMM kernels for A in e4m3 and B in e5m2: the kernels of gemm_inst_fp8.hip with one format field of their
// MFMAs set.  The deeper-pipeline variants of the small tiles are left out: such problems take the two-stage kernels.
// (One translation unit per mixture: both in one file crash this compiler in its first function passes.)
#include "gemm_variants.h"

namespace tb {

const Variant g_variants_e4e5[] = {
    make_variant_w4<W4Tile<DT_E4E5>>(),
    make_variant<Tile<DT_E4E5, 256, 256, 128, 2, 4, LAY_K, LAY_K, 1, true, 2>>(),
    make_variant<Tile<DT_E4E5, 128, 128, 128, 2, 2, LAY_K, LAY_K, 2, true, 2>>(),
    make_variant<Tile<DT_E4E5, 64, 64, 128, 2, 2, LAY_K, LAY_K, 4, true, 2>>(),
    make_variant<Tile<DT_E4E5, 32, 128, 256, 1, 4, LAY_K, LAY_K, 1, true, 3>>(),
    make_variant<Tile<DT_E4E5, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, false, 2>>(),
};
const int g_num_variants_e4e5 = sizeof(g_variants_e4e5) / sizeof(Variant);

}  // namespace tb
