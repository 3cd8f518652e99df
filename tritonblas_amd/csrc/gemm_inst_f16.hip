// f16 tile GEMM kernels: every tile shape for the four operand layout combinations, plus one
// element-wise-gather kernel for operands the vector loaders cannot address.
#include "gemm_variants.h"

namespace tb {

#define TB_LAYOUTS(BM, BN, WM, WN, MINB)                                              \
  make_variant<Tile<DT_F16, BM, BN, 128, WM, WN, LAY_K, LAY_K, MINB, true, 2>>(),      \
  make_variant<Tile<DT_F16, BM, BN, 128, WM, WN, LAY_K, LAY_M, MINB, true, 2>>(),      \
  make_variant<Tile<DT_F16, BM, BN, 128, WM, WN, LAY_M, LAY_K, MINB, true, 2>>(),      \
  make_variant<Tile<DT_F16, BM, BN, 128, WM, WN, LAY_M, LAY_M, MINB, true, 2>>()

const Variant g_variants_f16[] = {
    // hand-scheduled 4-wave kernel (K-major operands): taken when K is a multiple of two K steps and no Stream-K tail is asked for
    make_variant_w4<W4Tile<DT_F16>>(),
    TB_LAYOUTS(256, 256, 2, 4, 1),
    TB_LAYOUTS(128, 128, 2, 2, 2),
    TB_LAYOUTS(64, 64, 2, 2, 4),
    // deeper copy pipelines of the small tile for problems with few tiles per CU (each K step then
    // waits less for its copy; fewer workgroups fit a CU)
    make_variant<Tile<DT_F16, 64, 64, 128, 2, 2, LAY_K, LAY_K, 3, true, 3>>(),
    make_variant<Tile<DT_F16, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, true, 4>>(),
    // a handful of rows against a long K: short, wide, deep tile with three copy stages
    make_variant<Tile<DT_F16, 32, 128, 256, 1, 4, LAY_K, LAY_K, 1, true, 3>>(),
    make_variant<Tile<DT_F16, 32, 128, 256, 1, 4, LAY_K, LAY_M, 1, true, 2>>(),
    make_variant<Tile<DT_F16, 32, 128, 256, 1, 4, LAY_M, LAY_K, 1, true, 2>>(),
    make_variant<Tile<DT_F16, 32, 128, 256, 1, 4, LAY_M, LAY_M, 1, true, 2>>(),
    make_variant<Tile<DT_F16, 64, 64, 128, 2, 2, LAY_K, LAY_K, 2, false, 2>>(),
};
const int g_num_variants_f16 = sizeof(g_variants_f16) / sizeof(Variant);

}  // namespace tb
