// out[i] = table[in[i]] for 8-bit tensors: any elementwise function between two quantized
// tensors (dequantize -> activation -> quantize) collapses to a 256-entry table, because its
// input takes at most 256 values.  HBM-bound, 2 bytes per element; the table sits in LDS.
#include "dq8_common.h"
#include "disc_q8.h"

namespace dq8 {
namespace {

constexpr int kThreads = 256;
typedef unsigned vu4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ unsigned map4(const uint8_t* t, unsigned w) {
  return (unsigned)t[w & 0xff] | ((unsigned)t[(w >> 8) & 0xff] << 8) |
         ((unsigned)t[(w >> 16) & 0xff] << 16) | ((unsigned)t[w >> 24] << 24);
}

// 16 bytes per thread, one sweep; `table` is indexed by the byte's bit pattern
// (results leave with the streaming hint, a kilobyte per store instruction:
// [65536,4096] 89.8 -> 74.7 us, 7.2 TB/s; [4096,4096] 6.0 -> 4.8 us)
__global__ void __launch_bounds__(kThreads)
lut_u8_v16(const vu4* __restrict__ in, vu4* __restrict__ out, int64_t n16,
           const uint8_t* __restrict__ table) {
  __shared__ uint8_t t[256];
  t[threadIdx.x] = table[threadIdx.x];
  __syncthreads();
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n16; i += stride) {
    const vu4 v = in[i];
    const vu4 r = (vu4){map4(t, v[0]), map4(t, v[1]), map4(t, v[2]), map4(t, v[3])};
    __builtin_nontemporal_store(r, &out[i]);
  }
}

__global__ void __launch_bounds__(kThreads)
lut_u8_scalar(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int64_t begin, int64_t n,
              const uint8_t* __restrict__ table) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += stride)
    out[i] = table[in[i]];
}

}  // namespace
}  // namespace dq8

using namespace dq8;

extern "C" int dq8_lut8(const void* in, void* out, int64_t n, const void* table, void* stream) {
  clear_error();
  DQ8_REQUIRE(n >= 0, "dq8_lut8: negative size");
  if (n == 0) return 0;
  DQ8_REQUIRE(in && out && table, "dq8_lut8: null pointer");
  hipStream_t st = (hipStream_t)stream;
  int64_t done = 0;
  if (aligned(in, 16) && aligned(out, 16) && n >= 16) {
    const int64_t n16 = n / 16;
    int64_t blocks = ceil_div(n16, kThreads);
    if (blocks > (1LL << 22)) blocks = 1LL << 22;
    hipLaunchKernelGGL(lut_u8_v16, dim3((unsigned)blocks), dim3(kThreads), 0, st,
                       static_cast<const vu4*>(in), static_cast<vu4*>(out), n16,
                       static_cast<const uint8_t*>(table));
    done = n16 * 16;
  }
  if (done < n) {
    int64_t blocks = ceil_div(n - done, kThreads);
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(lut_u8_scalar, dim3((unsigned)blocks), dim3(kThreads), 0, st,
                       static_cast<const uint8_t*>(in), static_cast<uint8_t*>(out), done, n,
                       static_cast<const uint8_t*>(table));
  }
  return check_hip(hipGetLastError(), "dq8_lut8 launch");
}
