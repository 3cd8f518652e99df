// Skinny-M GEMM (decode shapes: a handful of activation rows against a long weight matrix).
//
// HBM-bound on B, which is read exactly once: every wave streams its B rows straight from global
// memory into MFMA operand registers (a lane's 16/32 bytes are contiguous along K, 16 lanes cover
// sixteen full 128-byte row segments), several K steps ahead, with no LDS and no barrier in the K
// loop.  The eight waves of a workgroup split K between them (intra-workgroup split-K) and reduce
// their fp32 partial tiles through LDS in a fixed order, so the result is deterministic and needs
// no global workspace.  A is small and comes from L2 / L1.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "gemm_device.h"
#include "skinny.h"

namespace tb {

template <int DT> struct SkT {
  static constexpr int LB = is_f8(DT) ? 32 : 16;        // bytes of K one lane feeds to one MFMA
  static constexpr int STEP = 4 * LB;                   // bytes of K per MFMA
  using frag_t = typename std::conditional<is_f8(DT), v8i, v4i>::type;
  __device__ static __forceinline__ frag_t load(const uint8_t* p) {
    if constexpr (is_f8(DT)) {
      v4i lo = *(const v4i*)p, hi = *(const v4i*)(p + 16);
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    } else {
      return *(const v4i*)p;
    }
  }
  __device__ static __forceinline__ v4f mma(frag_t x, frag_t y, v4f c) {
    if constexpr (DT == DT_F16) return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, x), __builtin_bit_cast(h8, y), c, 0, 0, 0);
    else if constexpr (DT == DT_BF16) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, x), __builtin_bit_cast(bf8, y), c, 0, 0, 0);
    else {
      constexpr int FMT = DT == DT_E5M2 ? 1 : 0;   // 0 = e4m3, 1 = e5m2, both operands
      return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(x, y, c, FMT, FMT, 0, 0, 0, 0);
    }
  }
};

template <int DT, int MT, int NT, int WAVES, int DEPTH>
__global__ __launch_bounds__(WAVES * 64) void skinny_kernel(const GemmParams p) {
  using S = SkT<DT>;
  using frag_t = typename S::frag_t;
  __shared__ __attribute__((aligned(16))) float red[WAVES][MT * NT][64][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * NT);
  constexpr int USZ = is_f8(DT) ? 1 : 2;

  // this wave's share of the K steps
  const int64_t kbytes = p.KU * USZ;
  const int steps = (int)(kbytes / S::STEP);
  const int q = steps / WAVES, rem = steps % WAVES;
  const int s0 = wave * q + min(wave, rem);
  const int ns = q + (wave < rem ? 1 : 0);

  const uint8_t* ap[MT];
  const uint8_t* bp[NT];
#pragma unroll
  for (int i = 0; i < MT; ++i) ap[i] = p.A + (int64_t)min(i * 16 + r, p.M - 1) * p.a_sr * USZ + (int64_t)s0 * S::STEP + g * S::LB;
#pragma unroll
  for (int j = 0; j < NT; ++j) bp[j] = p.B + (int64_t)min(n0 + j * 16 + r, p.N - 1) * p.b_sr * USZ + (int64_t)s0 * S::STEP + g * S::LB;

  v4f acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

  frag_t aq[DEPTH][MT], bq[DEPTH][NT];
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    if (d < ns) {
#pragma unroll
      for (int j = 0; j < NT; ++j) bq[d][j] = S::load(bp[j] + (int64_t)d * S::STEP);
#pragma unroll
      for (int i = 0; i < MT; ++i) aq[d][i] = S::load(ap[i] + (int64_t)d * S::STEP);
    }
  }
  for (int s = 0; s < ns; s += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (s + d < ns) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
          for (int j = 0; j < NT; ++j) acc[i][j] = S::mma(bq[d][j], aq[d][i], acc[i][j]);
        if (s + d + DEPTH < ns) {
#pragma unroll
          for (int j = 0; j < NT; ++j) bq[d][j] = S::load(bp[j] + (int64_t)(s + d + DEPTH) * S::STEP);
#pragma unroll
          for (int i = 0; i < MT; ++i) aq[d][i] = S::load(ap[i] + (int64_t)(s + d + DEPTH) * S::STEP);
        }
      }
    }
  }

  // reduce the WAVES partial tiles in wave order, then scale / bias / cast / store
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) *(v4f*)red[wave][i * NT + j][lane] = acc[i][j];
  __syncthreads();
  for (int t = wave; t < MT * NT; t += WAVES) {
    v4f v = *(const v4f*)red[0][t][lane];
    for (int w = 1; w < WAVES; ++w) v += *(const v4f*)red[w][t][lane];
    const int i = t / NT, j = t % NT;
    const int m = i * 16 + r;
    const int n = n0 + j * 16 + 4 * g;
    const int nvalid = p.N - n;
    if (m >= p.M || nvalid <= 0) continue;
    if (p.sa) {
      const float sa = p.sa[m];
#pragma unroll
      for (int e = 0; e < 4; ++e) if (e < nvalid) v[e] = v[e] * (sa * p.sb[n + e]);
    }
    if (p.bias) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (e < nvalid) v[e] += load_as_f32(p.bias + (int64_t)(n + e) * p.bias_stride * (p.bias_type == DT_F32 ? 4 : 2), p.bias_type);
    }
    const int64_t off = (int64_t)m * p.c_sm + (int64_t)n * p.c_sn;
    if (p.c_type == DT_BF16) store4<DT_BF16>(p.C, off, p.c_sn, v, nvalid, p.c_vec);
    else if (p.c_type == DT_F16) store4<DT_F16>(p.C, off, p.c_sn, v, nvalid, p.c_vec);
    else store4<DT_F32>(p.C, off, p.c_sn, v, nvalid, p.c_vec);
  }
}

template <int DT, int MT, int NT, int DEPTH>
static hipError_t launch_nt(const GemmParams& p, hipStream_t stream) {
  constexpr int WAVES = 8;
  const int grid = (p.N + 16 * NT - 1) / (16 * NT);
  hipLaunchKernelGGL((skinny_kernel<DT, MT, NT, WAVES, DEPTH>), dim3(grid), dim3(WAVES * 64), 0, stream, p);
  return hipGetLastError();
}

// Every workgroup reads all of A (from L2), so its cost per weight byte halves when a workgroup owns
// 64 columns instead of 32 -- worth it once 64-column workgroups still outnumber the CUs well
// (measured on 256 CUs: N = 28672, K = 8192, M = 32: 70 us -> 48 us; N = 8192 would leave half the CUs idle).
template <int DT, int MT>
static hipError_t launch_mt(const GemmParams& p, hipStream_t stream) {
  if (p.N >= 64 * 384) return launch_nt<DT, MT, 4, 2>(p, stream);
  return launch_nt<DT, MT, 2, 4>(p, stream);
}

template <int DT>
static hipError_t launch_dt(const GemmParams& p, hipStream_t stream) {
  if (p.M <= 16) return launch_mt<DT, 1>(p, stream);
  if (p.M <= 32) return launch_mt<DT, 2>(p, stream);
  return launch_mt<DT, 4>(p, stream);
}

// (operands of two different 8-bit float formats stay on the tile kernels: this compiler crashes on a translation unit
// that holds MFMAs of both mixtures, and a streaming kernel per mixture in files of their own is not worth two more)
bool skinny_supported(int dt, int64_t m) {
  return m <= SKINNY_MAX_M && (dt == DT_FP8 || dt == DT_E5M2 || dt == DT_F16 || dt == DT_BF16);
}

int skinny_k_step_units(int dt) { return is_f8(dt) ? 128 : 32; }

hipError_t launch_skinny(const GemmParams& p, int dt, hipStream_t stream) {
  if (dt == DT_FP8) return launch_dt<DT_FP8>(p, stream);
  if (dt == DT_E5M2) return launch_dt<DT_E5M2>(p, stream);
  if (dt == DT_F16) return launch_dt<DT_F16>(p, stream);
  return launch_dt<DT_BF16>(p, stream);
}

}  // namespace tb
