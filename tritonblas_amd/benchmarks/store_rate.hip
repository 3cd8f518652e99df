// How fast can the CUs write a C tile?  A stand-alone probe of the vector store path (no library code):
// every workgroup (4 waves) writes 14 tiles of 256 rows x 512 bytes, the bytes a 256x256 bf16 output tile
// has, in the lane pattern of the 4-wave GEMM epilogue (16 rows x 64 bytes per instruction) or in whole
// cache lines (8 rows x 128 bytes per instruction), with 1 .. 256 workgroups (one per CU), to distinct
// tiles of a 8192 x 28672 bf16 matrix or always to the same tile per workgroup (the lines then stay in L2).
//
//   hipcc --offload-arch=gfx950 -O3 -o /tmp/store_rate tritonblas_amd/benchmarks/store_rate.hip && /tmp/store_rate
//
// Prints, per case, the time per tile and the bytes per second over all workgroups.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef int v4i __attribute__((ext_vector_type(4)));
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

constexpr long ROWS = 8192, ROW_BYTES = 57344;            // 28672 bf16 per row
constexpr int TILES_N = (int)(ROW_BYTES / 512), TILES = 14;

// wave w of a workgroup writes rows (w / 2) * 128 .. + 127, byte columns (w % 2) * 256 .. + 255 of each tile
template <bool WHOLE_LINES>
__global__ __launch_bounds__(256, 1) void store_tiles(uint8_t* C, int same_tile) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  v4i val = {lane, wave, (int)blockIdx.x, 0};
  for (int t = 0; t < TILES; ++t) {
    const int tile = same_tile ? (int)blockIdx.x : (int)blockIdx.x + t * (int)gridDim.x;   // < 256 * 14 = 32 * 112 tiles
    uint8_t* base = C + ((long)(tile / TILES_N) * 256 + (wave >> 1) * 128) * ROW_BYTES + (long)(tile % TILES_N) * 512 + (wave & 1) * 256;
    val[3] = t;
    if (WHOLE_LINES) {
      const int r = lane >> 3, c = lane & 7;
#pragma unroll
      for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int q = 0; q < 2; ++q) *(v4i*)(base + (long)(i * 8 + r) * ROW_BYTES + q * 128 + c * 16) = val;
    } else {
      const int r = lane & 15, g = lane >> 4;
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) *(v4i*)(base + (long)(i * 16 + r) * ROW_BYTES + q * 64 + g * 16) = val;
    }
  }
}

template <bool WHOLE_LINES>
void run(uint8_t* C, int grid, int same_tile) {
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  for (int w = 0; w < 3; ++w) store_tiles<WHOLE_LINES><<<grid, 256>>>(C, same_tile);
  CK(hipDeviceSynchronize());
  const int reps = 20;
  CK(hipEventRecord(a));
  for (int w = 0; w < reps; ++w) store_tiles<WHOLE_LINES><<<grid, 256>>>(C, same_tile);
  CK(hipEventRecord(b));
  CK(hipDeviceSynchronize());
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, a, b));
  ms /= reps;
  const double bytes = (double)grid * TILES * 131072.0;
  printf("%4d workgroups  %-22s %-14s %6.2f us per tile  %6.2f TB/s  %5.1f GB/s per workgroup\n", grid,
         WHOLE_LINES ? "8 rows x 128 B / instr" : "16 rows x 64 B / instr", same_tile ? "same tile (L2)" : "distinct tiles", ms * 1e3 / TILES,
         bytes / ms / 1e9, bytes / grid / ms / 1e6);
  fflush(stdout);
  CK(hipEventDestroy(a));
  CK(hipEventDestroy(b));
}

int main() {
  uint8_t* C = nullptr;
  CK(hipMalloc(&C, (size_t)ROWS * ROW_BYTES));
  CK(hipMemset(C, 0, (size_t)ROWS * ROW_BYTES));
  const int grids[] = {1, 8, 64, 128, 256};
  for (int grid : grids)
    for (int same = 0; same < 2; ++same) {
      run<false>(C, grid, same);
      run<true>(C, grid, same);
    }
  CK(hipFree(C));
  return 0;
}
