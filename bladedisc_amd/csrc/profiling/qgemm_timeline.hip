// Timeline of the pipelined int8 GEMM kernel: when do its workgroups enter, see their
// first k tile land, finish the main loop and finish storing?  A standalone profiling
// program (not part of the library): it instantiates the kernel from the library's own
// header with the DQ8_TRACE_POINT hook defined, launches it on M = N = 4096 with three
// depths of K, once with four and once with eight waves per workgroup, and prints the
// stage times over all workgroups next to the hipEvent time of the launch.
//
// Build and run (bladedisc_amd/build.py: build_profiling_tools()):
//   hipcc -O3 -std=c++17 --offload-arch=gfx950 -ffp-contract=off \
//       -Xclang -target-feature -Xclang -packed-fp32-ops \
//       -Iinclude -Ibladedisc_amd/csrc/kernels \
//       -o bladedisc_amd/build/qgemm_timeline bladedisc_amd/csrc/profiling/qgemm_timeline.hip
//   bladedisc_amd/build/qgemm_timeline
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <vector>
#include <algorithm>
__device__ long long g_trace[4 * 4096];
#define DQ8_TRACE_POINT(i) do { if (threadIdx.x == 0) g_trace[4 * blockIdx.x + (i)] = wall_clock64(); } while (0)
#include "qgemm_pipelined.h"
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1);} } while (0)
using namespace dq8;
// WM x WN waves on the 256x256 tile: 2 x 2 (one wave per SIMD, wave tile 128x128) or 2 x 4
// (two per SIMD, wave tile 128x64)
template <int WM, int WN>
void run() {
  const int M = 4096, N = 4096;
  printf("---- %d waves per workgroup\n", WM * WN);
  for (int K : {128, 768, 4096}) {
    int8_t *A, *W, *out; float *sx, *sw, *so, *bias;
    CK(hipMalloc(&A, (size_t)M * K)); CK(hipMalloc(&W, (size_t)N * K)); CK(hipMalloc(&out, (size_t)M * N));
    CK(hipMalloc(&sx, 4)); CK(hipMalloc(&sw, 4 * N)); CK(hipMalloc(&so, 4)); CK(hipMalloc(&bias, 4 * N));
    { std::vector<int8_t> h((size_t)M * K); unsigned s = 7; for (auto& v : h) { s = s * 1664525u + 1013904223u; v = (int8_t)(s >> 24); }
      CK(hipMemcpy(A, h.data(), h.size(), hipMemcpyHostToDevice)); CK(hipMemcpy(W, h.data(), h.size(), hipMemcpyHostToDevice));
      std::vector<float> f(N, 0.01f); CK(hipMemcpy(sw, f.data(), 4 * N, hipMemcpyHostToDevice)); CK(hipMemcpy(bias, f.data(), 4 * N, hipMemcpyHostToDevice));
      float one = 0.02f, o = 30.f; CK(hipMemcpy(sx, &one, 4, hipMemcpyHostToDevice)); CK(hipMemcpy(so, &o, 4, hipMemcpyHostToDevice)); }
    MainParams p = {};
    p.A = A; p.W = W; p.lda = K; p.ldw = K; p.M = M; p.N = N; p.K = K; p.tiles_m = M / 256; p.tiles_n = N / 256;
    p.epi.out = out; p.epi.ldo = N; p.epi.M = M; p.epi.N = N; p.epi.bias = bias; p.epi.bias_kind = DQ8_BIAS_F32;
    p.epi.sx = sx; p.epi.sw = sw; p.epi.so = so; p.epi.sx_stride = 0; p.epi.sw_stride = 1; p.epi.so_stride = 0; p.epi.zo = 0;
    p.epi.vec_store = 1; p.epi.vec_store16 = 1;
    auto kern = qgemm_pipe_kernel<256, 256, WM, WN, 1, false, DQ8_EPI_REQUANT_GPU>;
    CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 131072));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    for (int r = 0; r < 3; ++r) hipLaunchKernelGGL(kern, dim3(256), dim3(WM * WN * 64), 131072, 0, p);
    CK(hipDeviceSynchronize());
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL(kern, dim3(256), dim3(WM * WN * 64), 131072, 0, p);
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    std::vector<long long> t(4 * 256);
    CK(hipMemcpyFromSymbol(t.data(), HIP_SYMBOL(g_trace), t.size() * 8));
    long long first = t[0];
    for (int b = 0; b < 256; ++b) first = std::min(first, t[4 * b]);
    double st[4][3];
    for (int i = 0; i < 4; ++i) {
      std::vector<double> v; for (int b = 0; b < 256; ++b) v.push_back((t[4 * b + i] - first) / 100.0);
      std::sort(v.begin(), v.end()); st[i][0] = v.front(); st[i][1] = v[128]; st[i][2] = v.back();
    }
    printf("K=%d  event %.1f us | us since first workgroup entered (min / median / max over 256 workgroups):\n", K, ms * 1e3);
    const char* names[4] = {"entry", "tile 0 landed", "main loop done", "stored, exit"};
    for (int i = 0; i < 4; ++i) printf("   %-16s %6.2f %6.2f %6.2f\n", names[i], st[i][0], st[i][1], st[i][2]);
    CK(hipFree(A)); CK(hipFree(W)); CK(hipFree(out));
  }
}

int main() {
  run<2, 2>();
  run<2, 4>();
  return 0;
}
