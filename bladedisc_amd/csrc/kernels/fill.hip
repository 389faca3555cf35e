// dst[0 .. bytes) = (uint8_t)value as an ordinary kernel launch: what the runtime's memset
// service issues instead of hipMemsetAsync, so that a program whose execution is captured
// into a HIP graph records a kernel node (memset nodes recorded into captured graphs have
// replayed wrongly on this hardware).  HBM-bound, 1 byte written per byte.
#include "dq8_common.h"
#include "disc_q8.h"

namespace dq8 {
namespace {

constexpr int kThreads = 256;
typedef unsigned vu4 __attribute__((ext_vector_type(4)));

// bytes [head, head + 16 n16) in 16-byte stores (dst + head is 16-byte aligned); the `head`
// bytes before and the `tail` bytes after by the first threads of block 0
__global__ void __launch_bounds__(kThreads)
fill_kernel(uint8_t* __restrict__ dst, unsigned word, int head, int64_t n16, int tail) {
  vu4* body = reinterpret_cast<vu4*>(dst + head);
  const vu4 v = {word, word, word, word};
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n16; i += stride) body[i] = v;
  if (blockIdx.x == 0) {
    const int t = threadIdx.x;
    if (t < head) dst[t] = (uint8_t)word;
    if (t >= 16 && t - 16 < tail) dst[head + n16 * 16 + (t - 16)] = (uint8_t)word;
  }
}

}  // namespace
}  // namespace dq8

using namespace dq8;

extern "C" int dq8_fill(void* dst, int value, size_t bytes, void* stream) {
  clear_error();
  if (bytes == 0) return 0;
  DQ8_REQUIRE(dst != nullptr, "dq8_fill: null pointer");
  const uintptr_t a = reinterpret_cast<uintptr_t>(dst);
  size_t head = (16 - (a & 15)) & 15;
  if (head > bytes) head = bytes;
  const int64_t n16 = (int64_t)((bytes - head) / 16);
  const int tail = (int)(bytes - head - (size_t)n16 * 16);
  const unsigned b = (unsigned)value & 0xffu;
  const unsigned word = b | (b << 8) | (b << 16) | (b << 24);
  int64_t blocks = ceil_div(n16 > 0 ? n16 : 1, kThreads);
  if (blocks > (1LL << 20)) blocks = 1LL << 20;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream,
                     static_cast<uint8_t*>(dst), word, (int)head, n16, tail);
  return check_hip(hipGetLastError(), "dq8_fill launch");
}
