// How fast can the matrix cores go on this part, and what does the data do to it?
// A standalone profiling program (not part of the library).  Each workgroup (4 waves, one
// per SIMD) runs the MFMA stream of the 256x256x128 GEMM tile -- 64 v_mfma_i32_32x32x32_i8
// per wave per "tile", 16 accumulator fragments -- on operands that stay in registers: no
// loads, no LDS, nothing but the matrix pipe.  It reports the rate and the shader clock
// actually delivered (clock64() ticks per wall_clock64() tick), for operands that are all
// equal and for random operands, with 8, 64 and all 256 CUs busy.
//
// Build and run (bladedisc_amd/build.py: build_profiling_tools()):
//   hipcc -O3 -std=c++17 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops \
//       -o bladedisc_amd/build/mfma_power_probe bladedisc_amd/csrc/profiling/mfma_power_probe.hip
//   bladedisc_amd/build/mfma_power_probe
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

#define CK(x)                                                        \
  do {                                                               \
    hipError_t e = (x);                                              \
    if (e != hipSuccess) {                                           \
      printf("%s: %s\n", #x, hipGetErrorString(e));                  \
      exit(1);                                                       \
    }                                                                \
  } while (0)

template <bool RANDOM>
__global__ void __launch_bounds__(256) mfma_loop(int tiles, int* sink, long long* clk) {
  const long long c0 = clock64(), w0 = wall_clock64();
  const int lane = threadIdx.x & 63;
  v16i acc[4][4];
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
  v4i fa[2][4], fb[2][4];
  for (int s = 0; s < 2; ++s)
    for (int i = 0; i < 4; ++i) {
      if (RANDOM) {
        unsigned h = (lane * 2654435761u) ^ (i * 40503u) ^ (s * 977u) ^ (blockIdx.x * 7919u) ^
                     (threadIdx.x * 31u);
        h *= 2246822519u;
        fa[s][i] = (v4i){(int)h, (int)(h * 3266489917u), (int)(h * 668265263u), (int)(h * 374761393u)};
        h = (h ^ 0x9e3779b9u) * 2246822519u;
        fb[s][i] = (v4i){(int)h, (int)(h * 3266489917u), (int)(h * 668265263u), (int)(h * 374761393u)};
      } else {
        fa[s][i] = (v4i){0x01010101, 0x01010101, 0x01010101, 0x01010101};
        fb[s][i] = fa[s][i];
      }
    }
  for (int t = 0; t < tiles; ++t) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ks & 1][j], fa[ks & 1][i], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  int s = 0;
  for (int i = 0; i < 4; ++i)
    for (int j = 0; j < 4; ++j)
      for (int v = 0; v < 16; ++v) s += acc[i][j][v];
  if (s == 0x12345678) sink[threadIdx.x] = s;   // keeps the accumulators alive
  if (threadIdx.x == 0) {
    clk[2 * blockIdx.x] = clock64() - c0;
    clk[2 * blockIdx.x + 1] = wall_clock64() - w0;
  }
}

template <bool RANDOM>
void run(const char* what, int grid, int tiles, int* sink, long long* clk) {
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int r = 0; r < 2; ++r) hipLaunchKernelGGL(mfma_loop<RANDOM>, dim3(grid), dim3(256), 0, 0, tiles, sink, clk);
  CK(hipEventRecord(e0));
  const int reps = 5;
  for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(mfma_loop<RANDOM>, dim3(grid), dim3(256), 0, 0, tiles, sink, clk);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  ms /= reps;
  long long h[2];
  CK(hipMemcpy(h, clk, sizeof(h), hipMemcpyDeviceToHost));
  int wall_khz = 0;
  CK(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, 0));
  const double ops = (double)grid * 4 * tiles * 64 * 65536.0;
  printf("%-18s %3d workgroups: %7.1f us  %7.1f TOP/s  %.2f us per 256x256x128 tile  shader clock %.0f MHz\n",
         what, grid, ms * 1e3, ops / ms / 1e9, ms * 1e3 / tiles, (double)h[0] / h[1] * wall_khz / 1e3);
}

int main() {
  int* sink;
  long long* clk;
  CK(hipMalloc(&sink, 4096));
  CK(hipMalloc(&clk, 2 * 256 * sizeof(long long)));
  const int tiles = 128;
  for (int rep = 0; rep < 2; ++rep)
    for (int grid : {8, 64, 256}) {
      run<false>("equal operands", grid, tiles, sink, clk);
      run<true>("random operands", grid, tiles, sink, clk);
    }
  return 0;
}
