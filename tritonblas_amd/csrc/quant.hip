// Fused blockwise Hadamard-32 rotation + MXFP4 quantisation (e2m1 codes, E8M0 scale per 32 values).
//
// HBM-bound: every input element is read once (16-byte loads, a wave covers 1 KiB of a row) and
// 4.25 bits per element are written; loads and stores are marked non-temporal (nothing is touched
// twice), which together with the division-free index arithmetic is worth 15 % on 8192x16384 bf16.  Four neighbouring lanes own one 32-value block (8 values
// each); the butterfly stages with stride 8 and 16 and the block maximum cross lanes with
// quad-permute DPP moves, so nothing goes through LDS.
//
// Bit-level definition of the quantiser (must stay integer-exact):
//   amax -> (bits + 0x200000) & 0xFF800000 -> e = exponent - 2, clamped to [-127, 127]
//   scale byte = (e + 127) & 0xFF ; q = x * 2^-e ; code = round-half-up-in-magnitude(q), saturated to 6.0
// The last step runs on v_cvt_scalef32_pk_fp4_f32 (two values per instruction); see the tie handling below.
// This file is compiled with -ffp-contract=off: the rotation is fp32 adds/subs and one multiply.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>
#include "quant.h"

namespace tb {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float dpp_xor1(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_xor2(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
}

template <int XT>
__device__ __forceinline__ void load8(const uint8_t* p, float (&v)[8]) {
  if constexpr (XT == QT_F32) {
    const v4f a = __builtin_nontemporal_load((const v4f*)p);
    const v4f b = __builtin_nontemporal_load((const v4f*)(p + 16));
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
    const v4i raw = __builtin_nontemporal_load((const v4i*)p);
    const uint32_t w[4] = {(uint32_t)raw.x, (uint32_t)raw.y, (uint32_t)raw.z, (uint32_t)raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (XT == QT_BF16) {
        v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
        v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
      } else {
        v[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xffffu));
        v[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
      }
    }
  }
}

// MAGIC: the item count fits 31 bits and p.div_magic / p.div_shift divide by the items per row
template <int XT, bool HAD, int UNROLL, bool MAGIC>
__global__ __launch_bounds__(256) void quant_kernel(const QuantParams p) {
  const int64_t nc = p.n >> 3;  // 8-value items per row
  const int64_t items = p.m * nc;
  const int64_t base = ((int64_t)blockIdx.x * UNROLL) * 256 + threadIdx.x;
  const int sub = threadIdx.x & 3;
  constexpr int XB = (XT == QT_F32) ? 4 : 2;

  float v[UNROLL][8];
  int64_t row[UNROLL], col[UNROLL];
  bool ok[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    int64_t it = base + (int64_t)u * 256;
    ok[u] = it < items;
    if (!ok[u]) it = items - 1;  // keep the quad complete; nothing is stored for it
    if constexpr (MAGIC) {
      const uint32_t it32 = (uint32_t)it;
      const uint32_t q = p.div_shift < 0 ? it32 : (__umulhi(it32, p.div_magic) >> p.div_shift);
      row[u] = q;
      col[u] = it32 - q * (uint32_t)nc;
    } else {
      row[u] = it / nc;
      col[u] = it - row[u] * nc;
    }
    load8<XT>(p.x + (row[u] * p.x_stride + col[u] * 8) * XB, v[u]);
  }

#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    float(&x)[8] = v[u];
    if constexpr (HAD) {
#pragma unroll
      for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if ((i & h) == 0) {
            float a = x[i], b = x[i + h];
            x[i] = a + b;
            x[i + h] = a - b;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {  // stride 8: partner is lane ^ 1
        float o = dpp_xor1(x[i]);
        x[i] = (sub & 1) ? (o - x[i]) : (x[i] + o);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {  // stride 16: partner is lane ^ 2
        float o = dpp_xor2(x[i]);
        x[i] = (sub & 2) ? (o - x[i]) : (x[i] + o);
      }
      const float inv_sqrt32 = __builtin_bit_cast(float, 0x3E3504F3u);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = x[i] * inv_sqrt32;
    }
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(x[i]));
    amax = fmaxf(amax, dpp_xor1(amax));
    amax = fmaxf(amax, dpp_xor2(amax));

    uint32_t ab = (__builtin_bit_cast(uint32_t, amax) + 0x200000u) & 0xFF800000u;
    int field = (int)((ab >> 23) & 0xFFu);
    int e = field - 129;
    if (field == 0) e = -127;
    if (field == 255) e = 127;
    e = e < -127 ? -127 : (e > 127 ? 127 : e);
    // 2^-e as fp32 bits: normal for -e >= -126, the sub-normal 2^-127 for e = 127
    uint32_t qb = (e == 127) ? 0x00400000u : ((uint32_t)(127 - e) << 23);
    const float qs = __builtin_bit_cast(float, qb);
    // e2m1 conversion on the hardware converter.  It rounds to nearest-even; the quantiser's rule is
    // round-half-up in magnitude.  Setting the lowest fp32 mantissa bit moves every exact tie just
    // above the tie point and changes no other rounding decision (tie points have zero low bits).
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const float q0 = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x[i] * qs) | 1u);
      const float q1 = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x[i + 1] * qs) | 1u);
      if (i == 0) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, q0, q1, 1.0f, 0);
      if (i == 2) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, q0, q1, 1.0f, 1);
      if (i == 4) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, q0, q1, 1.0f, 2);
      if (i == 6) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, q0, q1, 1.0f, 3);
    }
    if (ok[u]) {
      __builtin_nontemporal_store(packed, (uint32_t*)(p.codes + row[u] * p.codes_stride + col[u] * 4));
      if (sub == 0) p.scales[row[u] * p.scales_stride + (col[u] >> 2)] = (uint8_t)((e + 127) & 0xFF);
    }
  }
}

template <int XT, bool HAD>
static hipError_t launch_t(const QuantParams& p0, bool force_div64, hipStream_t stream) {
  constexpr int UNROLL = 4;
  QuantParams p = p0;
  const int64_t nc = p.n >> 3;
  const int64_t items = p.m * nc;
  const int64_t per_block = 256 * UNROLL;
  const int64_t grid = (items + per_block - 1) / per_block;
  // (force_div64: testing hook, takes the kernel for 2^31 items and more at any size)
  if (items < (1ll << 31) && !force_div64) {
    // floor(i / nc) for i < 2^31: with l = ceil(log2 nc) and magic = floor(2^(31+l) / nc) + 1 < 2^32,
    // (i * magic) >> (31 + l) is exact; the kernel takes the high product word and shifts by l - 1
    int l = 0;
    while ((1ll << l) < nc) ++l;
    if (l == 0) { p.div_magic = 0; p.div_shift = -1; }
    else { p.div_magic = (uint32_t)(((1ull << (31 + l)) / (uint64_t)nc) + 1); p.div_shift = l - 1; }
    hipLaunchKernelGGL((quant_kernel<XT, HAD, UNROLL, true>), dim3((unsigned)grid), dim3(256), 0, stream, p);
  } else {
    hipLaunchKernelGGL((quant_kernel<XT, HAD, UNROLL, false>), dim3((unsigned)grid), dim3(256), 0, stream, p);
  }
  return hipGetLastError();
}

hipError_t launch_quant(const QuantParams& p, int x_type, bool hadamard, bool force_div64, hipStream_t stream) {
  if (x_type == QT_BF16) return hadamard ? launch_t<QT_BF16, true>(p, force_div64, stream) : launch_t<QT_BF16, false>(p, force_div64, stream);
  if (x_type == QT_F16) return hadamard ? launch_t<QT_F16, true>(p, force_div64, stream) : launch_t<QT_F16, false>(p, force_div64, stream);
  return hadamard ? launch_t<QT_F32, true>(p, force_div64, stream) : launch_t<QT_F32, false>(p, force_div64, stream);
}

}  // namespace tb
