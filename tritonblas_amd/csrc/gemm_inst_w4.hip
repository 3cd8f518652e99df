// The hand-scheduled 4-wave 256x256 kernels of MXFP4, bf16, fp16 and int8 (see gemm_w4.h); those of the 8-bit float
// formats are compiled in gemm_inst_w4f8.hip.
#include "gemm_w4.h"

namespace tb {

const void* w4_kernel_f8(int dt, bool sk);

const void* w4_kernel(int dt) {
  if (is_f8(dt)) return w4_kernel_f8(dt, false);
  if (dt == DT_FP4) return (const void*)&gemm_kernel_w4<W4Tile<DT_FP4>>;
  if (dt == DT_BF16) return (const void*)&gemm_kernel_w4<W4Tile<DT_BF16>>;
  if (dt == DT_F16) return (const void*)&gemm_kernel_w4<W4Tile<DT_F16>>;
  if (dt == DT_I8) return (const void*)&gemm_kernel_w4<W4Tile<DT_I8>>;
  return nullptr;
}

// the same kernels with the Stream-K tail
const void* w4_kernel_sk(int dt) {
  if (is_f8(dt)) return w4_kernel_f8(dt, true);
  if (dt == DT_FP4) return (const void*)&gemm_kernel_w4<W4Tile<DT_FP4>, true>;
  if (dt == DT_BF16) return (const void*)&gemm_kernel_w4<W4Tile<DT_BF16>, true>;
  if (dt == DT_F16) return (const void*)&gemm_kernel_w4<W4Tile<DT_F16>, true>;
  if (dt == DT_I8) return (const void*)&gemm_kernel_w4<W4Tile<DT_I8>, true>;
  return nullptr;
}

}  // namespace tb
