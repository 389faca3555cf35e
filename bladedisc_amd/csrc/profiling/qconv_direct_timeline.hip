// Timeline of the direct 3x3 convolution kernel: when do its workgroups enter, see their
// input patch land, finish the k loop and finish storing?  A standalone profiling program
// (not part of the library): it instantiates the kernel from the library's own header with
// the DQ8_TRACE_POINT hook defined, launches it on two ResNet-shaped layers (batch 32) and
// prints the stage times over all workgroups next to the hipEvent time of the launch.
//
// Build and run (bladedisc_amd/build.py: build_profiling_tools()):
//   hipcc -O3 -std=c++17 --offload-arch=gfx950 -ffp-contract=off \
//       -Xclang -target-feature -Xclang -packed-fp32-ops \
//       -Iinclude -Ibladedisc_amd/csrc/kernels \
//       -o bladedisc_amd/build/qconv_direct_timeline \
//       bladedisc_amd/csrc/profiling/qconv_direct_timeline.hip
//   bladedisc_amd/build/qconv_direct_timeline
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>
__device__ long long g_trace[4 * 8192];
#define DQ8_TRACE_POINT(i) \
  do { if (threadIdx.x == 0) g_trace[4 * blockIdx.x + (i)] = wall_clock64(); } while (0)
#include "qconv_direct.h"
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1); } } while (0)
using namespace dq8;

constexpr int kStages = 4;

template <int BM, int BN, int WM, int WN>
void run(int NB, int H, int Ci, int Co) {
  int8_t *in, *w, *out;
  float *sx, *sw, *so, *bias;
  const size_t in_b = (size_t)NB * H * H * Ci, w_b = (size_t)Co * 9 * Ci, o_b = (size_t)NB * H * H * Co;
  CK(hipMalloc(&in, in_b)); CK(hipMalloc(&w, w_b)); CK(hipMalloc(&out, o_b));
  CK(hipMalloc(&sx, 4)); CK(hipMalloc(&sw, 4 * Co)); CK(hipMalloc(&so, 4)); CK(hipMalloc(&bias, 4 * Co));
  {
    std::vector<int8_t> h(std::max(in_b, w_b));
    unsigned s = 7;
    for (auto& v : h) { s = s * 1664525u + 1013904223u; v = (int8_t)(s >> 24); }
    CK(hipMemcpy(in, h.data(), in_b, hipMemcpyHostToDevice));
    CK(hipMemcpy(w, h.data(), w_b, hipMemcpyHostToDevice));
    std::vector<float> f(Co, 0.01f);
    CK(hipMemcpy(sw, f.data(), 4 * Co, hipMemcpyHostToDevice));
    CK(hipMemcpy(bias, f.data(), 4 * Co, hipMemcpyHostToDevice));
    const float a = 0.02f, o = 30.f;
    CK(hipMemcpy(sx, &a, 4, hipMemcpyHostToDevice));
    CK(hipMemcpy(so, &o, 4, hipMemcpyHostToDevice));
  }
  DirectConvParams p = {};
  p.in = in; p.w = w; p.NB = NB; p.H = H; p.Wd = H; p.Ci = Ci; p.Co = Co; p.Ho = H; p.Wo = H;
  p.pad_t = 1; p.pad_l = 1;
  while ((1 << p.log2_ci) < Ci) ++p.log2_ci;
  const int hw = H * H;
  p.tiles_per_image = (hw + BM - 1) / BM;
  p.tiles_n = (Co + BN - 1) / BN;
  int span = 0;
  for (int t = 0; t < p.tiles_per_image; ++t) {
    const int first = t * BM, last = std::min(first + BM, hw) - 1;
    span = std::max(span, last / H - first / H + 1);
  }
  p.patch_bytes = ((span + 2) * (H + 2) * Ci + 1023) / 1024 * 1024;
  p.in_bytes = (int64_t)in_b;
  p.epi.out = out; p.epi.ldo = Co; p.epi.M = NB * hw; p.epi.N = Co;
  p.epi.bias = bias; p.epi.bias_kind = DQ8_BIAS_F32;
  p.epi.sx = sx; p.epi.sw = sw; p.epi.so = so;
  p.epi.sx_stride = 0; p.epi.sw_stride = 1; p.epi.so_stride = 0; p.epi.zo = 0;
  p.epi.vec_store = 1; p.epi.vec_store16 = 1;
  auto kern = qconv3x3_direct_kernel<BM, BN, WM, WN, kStages, DQ8_EPI_REQUANT_CPU>;
  CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  const int lds = p.patch_bytes + kStages * BN * 128;
  const int grid = NB * p.tiles_per_image * p.tiles_n;
  if (grid > 8192 || lds > 160 * 1024) { printf("shape does not fit this harness\n"); exit(1); }
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  for (int r = 0; r < 20; ++r) hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, 0, p);
  CK(hipDeviceSynchronize());
  CK(hipEventRecord(e0));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, 0, p);
  CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  std::vector<long long> t(4 * grid);
  CK(hipMemcpyFromSymbol(t.data(), HIP_SYMBOL(g_trace), t.size() * 8));
  long long first = t[0];
  for (int b = 0; b < grid; ++b) first = std::min(first, t[4 * b]);
  printf("conv %dx%dx%dx%d -> %d, tile %dx%d, %d workgroups, %d B of LDS each: hipEvent %.1f us\n",
         NB, H, H, Ci, Co, BM, BN, grid, lds, ms * 1e3);
  printf("  us since the first workgroup entered (min / median / max over the workgroups):\n");
  const char* names[4] = {"entry", "patch landed", "k loop done", "stored, exit"};
  for (int i = 0; i < 4; ++i) {
    std::vector<double> v;
    for (int b = 0; b < grid; ++b) v.push_back((t[4 * b + i] - first) / 100.0);   // 100 MHz clock
    std::sort(v.begin(), v.end());
    printf("   %-16s %6.2f %6.2f %6.2f\n", names[i], v.front(), v[grid / 2], v.back());
  }
  printf("  us a workgroup spends in each stage (min / median / max):\n");
  const char* stage_names[3] = {"entry -> patch", "k loop", "requant + store"};
  for (int i = 1; i < 4; ++i) {
    std::vector<double> v;
    for (int b = 0; b < grid; ++b) v.push_back((t[4 * b + i] - t[4 * b + i - 1]) / 100.0);
    std::sort(v.begin(), v.end());
    printf("   %-16s %6.2f %6.2f %6.2f\n", stage_names[i - 1], v.front(), v[grid / 2], v.back());
  }
  CK(hipFree(in)); CK(hipFree(w)); CK(hipFree(out));
  CK(hipFree(sx)); CK(hipFree(sw)); CK(hipFree(so)); CK(hipFree(bias));
}

int main() {
  run<256, 64, 4, 1>(32, 56, 64, 64);
  run<128, 64, 2, 2>(32, 28, 128, 128);
  return 0;
}
