// MXFP4 (e2m1 + E8M0 block-32 scales) tile GEMM kernels; operands are K-packed bytes.
#include "gemm_variants.h"

namespace tb {

const Variant g_variants_fp4[] = {
    // hand-scheduled 4-wave kernel: taken when K is a multiple of two K steps and no Stream-K tail is asked for
    make_variant_w4<W4Tile<DT_FP4>>(),
    make_variant<Tile<DT_FP4, 256, 256, 128, 2, 4, LAY_K, LAY_K, 1, true, 2>>(),
    make_variant<Tile<DT_FP4, 128, 128, 128, 2, 2, LAY_K, LAY_K, 2, true, 2>>(),
    make_variant<Tile<DT_FP4, 128, 128, 64, 2, 2, LAY_K, LAY_K, 2, true, 2>>(),
    make_variant<Tile<DT_FP4, 64, 64, 128, 2, 2, LAY_K, LAY_K, 4, true, 2>>(),
    make_variant<Tile<DT_FP4, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, false, 2>>(),
};
const int g_num_variants_fp4 = sizeof(g_variants_fp4) / sizeof(Variant);

}  // namespace tb
