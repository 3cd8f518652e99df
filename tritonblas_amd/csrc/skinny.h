// Host-visible entry of the skinny-M (decode) GEMM kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tb {

struct GemmParams;
constexpr int SKINNY_MAX_M = 64;

// true when the kernel exists for this element type and row count
bool skinny_supported(int dt, int64_t m);
// K must be a multiple of this many storage units
int skinny_k_step_units(int dt);
hipError_t launch_skinny(const GemmParams& p, int dt, hipStream_t stream);

}  // namespace tb
