// The hand-scheduled 4-wave 256x256 kernels (FP8 e4m3 and e5m2, MXFP4, bf16, fp16, int8), see gemm_w4.h.
#include "gemm_w4.h"

namespace tb {

const void* w4_kernel(int dt) {
  if (dt == DT_FP8) return (const void*)&gemm_kernel_w4<W4Tile<DT_FP8>>;
  if (dt == DT_E5M2) return (const void*)&gemm_kernel_w4<W4Tile<DT_E5M2>>;
  if (dt == DT_FP4) return (const void*)&gemm_kernel_w4<W4Tile<DT_FP4>>;
  if (dt == DT_BF16) return (const void*)&gemm_kernel_w4<W4Tile<DT_BF16>>;
  if (dt == DT_F16) return (const void*)&gemm_kernel_w4<W4Tile<DT_F16>>;
  if (dt == DT_I8) return (const void*)&gemm_kernel_w4<W4Tile<DT_I8>>;
  return nullptr;
}

// the same kernels with the Stream-K tail
const void* w4_kernel_sk(int dt) {
  if (dt == DT_FP8) return (const void*)&gemm_kernel_w4<W4Tile<DT_FP8>, true>;
  if (dt == DT_E5M2) return (const void*)&gemm_kernel_w4<W4Tile<DT_E5M2>, true>;
  if (dt == DT_FP4) return (const void*)&gemm_kernel_w4<W4Tile<DT_FP4>, true>;
  if (dt == DT_BF16) return (const void*)&gemm_kernel_w4<W4Tile<DT_BF16>, true>;
  if (dt == DT_F16) return (const void*)&gemm_kernel_w4<W4Tile<DT_F16>, true>;
  if (dt == DT_I8) return (const void*)&gemm_kernel_w4<W4Tile<DT_I8>, true>;
  return nullptr;
}

}  // namespace tb

#ifdef W4_LAB_TS
// measurement build: copies the timestamps of the last launch to the host (synchronises)
extern "C" int tb_lab_timestamps(unsigned long long* dst) {
  return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(tb::w4_lab_ts), sizeof(tb::w4_lab_ts));
}
#endif
