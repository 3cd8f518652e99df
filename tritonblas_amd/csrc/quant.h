// Host/device shared declarations of the MXFP4 quantisation kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tb {

enum : int { QT_F16 = 0, QT_BF16 = 1, QT_F32 = 4 };  // same numbering as the public element types

struct QuantParams {
  const uint8_t* x;
  uint8_t* codes;
  uint8_t* scales;
  int64_t m, n;
  int64_t x_stride;       // elements
  int64_t codes_stride;   // bytes
  int64_t scales_stride;  // bytes
  // item index -> (row, column) without a 64-bit division while the item count fits 31 bits:
  // row = mulhi(item, div_magic) >> div_shift (div_shift < 0: one item per row)
  uint32_t div_magic;
  int32_t div_shift;
};

hipError_t launch_quant(const QuantParams& p, int x_type, bool hadamard, bool force_div64, hipStream_t stream);

}  // namespace tb
