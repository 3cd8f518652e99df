// The hand-scheduled 4-wave 256x256 kernels of the 8-bit float formats: e4m3, e5m2 and the two mixtures (A in one
// format, B in the other).  See gemm_w4.h; gemm_inst_w4.hip hands out their addresses.
#include "gemm_w4.h"

namespace tb {

const void* w4_kernel_f8(int dt, bool sk) {
  if (dt == DT_FP8) return sk ? (const void*)&gemm_kernel_w4<W4Tile<DT_FP8>, true> : (const void*)&gemm_kernel_w4<W4Tile<DT_FP8>>;
  if (dt == DT_E5M2) return sk ? (const void*)&gemm_kernel_w4<W4Tile<DT_E5M2>, true> : (const void*)&gemm_kernel_w4<W4Tile<DT_E5M2>>;
  if (dt == DT_E4E5) return sk ? (const void*)&gemm_kernel_w4<W4Tile<DT_E4E5>, true> : (const void*)&gemm_kernel_w4<W4Tile<DT_E4E5>>;
  if (dt == DT_E5E4) return sk ? (const void*)&gemm_kernel_w4<W4Tile<DT_E5E4>, true> : (const void*)&gemm_kernel_w4<W4Tile<DT_E5E4>>;
  return nullptr;
}

}  // namespace tb

#ifdef W4_LAB_TS
// measurement build: copies the timestamps of the last launch to the host (synchronises)
extern "C" int tb_lab_timestamps(unsigned long long* dst) {
  return (int)hipMemcpyFromSymbol(dst, HIP_SYMBOL(tb::w4_lab_ts), sizeof(tb::w4_lab_ts));
}
#endif
