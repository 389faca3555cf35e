// Pieces shared by the bandwidth-bound elementwise kernels (quantize / dequantize in their
// mhlo_disc and TensorFlow forms): byte packing and the launch shapes of the three access
// patterns -- a linear sweep, [rows, channels] tiles with the channel on the last axis, and
// one (outer, channel) row per blockIdx.y.
#pragma once
#include <algorithm>
#include <cstdint>

#include "dq8_common.h"

namespace dq8 {

// Streaming loads and stores (the "non-temporal" hint): for tensors that are swept once.  Every
// wave instruction below covers whole 128-byte lines.
typedef float dq8_v4f_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void st_stream(float4* p, const float4& v) {
  __builtin_nontemporal_store((dq8_v4f_t){v.x, v.y, v.z, v.w}, reinterpret_cast<dq8_v4f_t*>(p));
}
__device__ __forceinline__ void st_stream(uint32_t* p, uint32_t v) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ float4 ld_stream(const float4* p) {
  const dq8_v4f_t v = __builtin_nontemporal_load(reinterpret_cast<const dq8_v4f_t*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint32_t ld_stream(const uint32_t* p) { return __builtin_nontemporal_load(p); }
namespace elementwise {

constexpr int kThreads = 256;

// A zero the compiler cannot see through.  Adding it to a workgroup-uniform index
// turns the parameter fetch into a vector load, which is issued together with the
// data load; as a scalar load it would be waited for (a cold miss, one per row) before
// the data load even starts.
__device__ __forceinline__ unsigned opaque_zero() {
  unsigned z;
  asm volatile("v_mov_b32 %0, 0" : "=v"(z));
  return z;
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
  return (uint32_t)(a & 0xff) | ((uint32_t)(b & 0xff) << 8) |
         ((uint32_t)(c & 0xff) << 16) | ((uint32_t)(d & 0xff) << 24);
}

// mhlo_disc.quantize of one element (R disc/transforms/disc_lower_quantize_and_dequantize.cc
// :77-94): divide, add the zero point, round, clamp, convert -- each a separately rounded f32
// operation (every file that includes this is compiled with -ffp-contract=off), the division
// a true IEEE division.  ROUND: 1 = half to even, 0 = half away from zero.
template <int ROUND>
__device__ __forceinline__ int quant_one(float x, float s, float z, float lo, float hi) {
  float t0 = x / s;
  float t1 = t0 + z;
  float t2 = ROUND == 1 ? rintf(t1) : roundf(t1);
  float t3 = fminf(fmaxf(t2, lo), hi);  // clamp; NaN -> lo like the CPU loop
  return (int)t3;
}

// Four quotients x / s for a divisor that is the same for a whole kernel, from its reciprocal
// y = 1.0f / s (a true division, done once): q0 = x y, r = fma(-q0, s, x), q = fma(r, y, q0).
// With y correctly rounded and q0 within an ulp of the quotient, r is exact and q is the
// correctly rounded x / s (Markstein's correction step) as long as nothing under- or
// overflows; the caller guarantees 2^-40 <= |s| <= 2^40, and an infinite or NaN x, or a q0
// that overflows, ends as NaN, in which case the four are divided for real.  Checked against
// x / s on the CPU for every one of the 2^32 values of x and 18 divisors (powers of two, all-ones
// and 1 + ulp significands, negative, 2^-23 .. 2^23): the same bits wherever 1/8 <= |x / s| <=
// 1024 and the same int8 after rounding (either mode) and clamping everywhere else
// (tests/native/div_by_constant_check.c runs a sample of that).
__device__ __forceinline__ float4 div4_by_constant(const float4& x, float s, float y) {
  float4 q;
  {
    const float a = x.x * y, b = x.y * y, c = x.z * y, d = x.w * y;
    q.x = __builtin_fmaf(__builtin_fmaf(-a, s, x.x), y, a);
    q.y = __builtin_fmaf(__builtin_fmaf(-b, s, x.y), y, b);
    q.z = __builtin_fmaf(__builtin_fmaf(-c, s, x.z), y, c);
    q.w = __builtin_fmaf(__builtin_fmaf(-d, s, x.w), y, d);
  }
  const float probe = (q.x + q.y) + (q.z + q.w);   // NaN if any is NaN (or +inf meets -inf)
  if (__builtin_expect(!(probe == probe) || __builtin_fabsf(probe) == __builtin_inff(), 0)) {
    q.x = x.x / s;
    q.y = x.y / s;
    q.z = x.z / s;
    q.w = x.w / s;
  }
  return q;
}

// The same with a divisor per component (per-channel scales on the last axis).
__device__ __forceinline__ float4 div4_by_constants(const float4& x, const float4& s, const float4& y) {
  float4 q;
  {
    const float a = x.x * y.x, b = x.y * y.y, c = x.z * y.z, d = x.w * y.w;
    q.x = __builtin_fmaf(__builtin_fmaf(-a, s.x, x.x), y.x, a);
    q.y = __builtin_fmaf(__builtin_fmaf(-b, s.y, x.y), y.y, b);
    q.z = __builtin_fmaf(__builtin_fmaf(-c, s.z, x.z), y.z, c);
    q.w = __builtin_fmaf(__builtin_fmaf(-d, s.w, x.w), y.w, d);
  }
  const float probe = (q.x + q.y) + (q.z + q.w);
  if (__builtin_expect(!(probe == probe) || __builtin_fabsf(probe) == __builtin_inff(), 0)) {
    q.x = x.x / s.x;
    q.y = x.y / s.y;
    q.z = x.z / s.z;
    q.w = x.w / s.w;
  }
  return q;
}

// Whether div4_by_constant may be used with divisor s.
__device__ __forceinline__ bool divisor_in_fast_range(float s) {
  const float a = __builtin_fabsf(s);
  return a >= 9.094947017729282e-13f && a <= 1099511627776.0f;   // 2^-40 .. 2^40
}

// quant_one from the quotient on (zero point 0)
template <int ROUND>
__device__ __forceinline__ int quant_from_quotient(float t0, float lo, float hi) {
  float t2 = ROUND == 1 ? rintf(t0) : roundf(t0);
  float t3 = fminf(fmaxf(t2, lo), hi);
  return (int)t3;
}

// Four quotients -> four int8 in one word, half-to-even rounding: clamp first (for integer
// bounds clamp(rne(t)) = rne(clamp(t)); v_med3_f32 returns the smaller bound for a NaN, as
// quant_one's fmaxf / fminf pair does), then one addition of 1.5 * 2^23 per value rounds to the
// nearest-even integer and leaves its two's-complement int8 in the low byte of the sum, which
// the sub-dword form of the add writes straight into its byte of the word.
// (lo, hi: integers in [-128, 255] -- the bounds of an 8-bit type or inside them)
__device__ __forceinline__ uint32_t quant4_pack_rne(const float4& t, float lo = -128.0f,
                                                    float hi = 127.0f) {
  const float c0 = __builtin_amdgcn_fmed3f(t.x, lo, hi);
  const float c1 = __builtin_amdgcn_fmed3f(t.y, lo, hi);
  const float c2 = __builtin_amdgcn_fmed3f(t.z, lo, hi);
  const float c3 = __builtin_amdgcn_fmed3f(t.w, lo, hi);
  const float magic = 12582912.0f;
  uint32_t word = __float_as_uint(c0 + magic);   // byte 0; bytes 1 .. 3 are replaced below
#if defined(__HIP_DEVICE_COMPILE__)
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(word) : "v"(c1), "v"(magic));
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(word) : "v"(c2), "v"(magic));
  asm("v_add_f32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
      : "+v"(word) : "v"(c3), "v"(magic));
#else
  word &= 0xffu;
  word |= (__float_as_uint(c1 + magic) & 0xffu) << 8;
  word |= (__float_as_uint(c2 + magic) & 0xffu) << 16;
  word |= (__float_as_uint(c3 + magic) & 0xffu) << 24;
#endif
  return word;
}

template <bool SIGNED>
__device__ __forceinline__ int4 unpack4(uint32_t w) {
  if (SIGNED)
    return make_int4((int8_t)(w & 0xff), (int8_t)((w >> 8) & 0xff), (int8_t)((w >> 16) & 0xff),
                     (int8_t)(w >> 24));
  return make_int4(w & 0xff, (w >> 8) & 0xff, (w >> 16) & 0xff, w >> 24);
}

inline int grid_for(int64_t work_items, int per_thread) {
  // enough blocks to cover the work with `per_thread` items per thread, capped at
  // 16 blocks per CU (256 CUs) so the grid-stride loops keep loads in flight
  int64_t blocks = dq8::ceil_div(work_items, (int64_t)kThreads * per_thread);
  if (blocks < 1) blocks = 1;
  if (blocks > 256 * 16) blocks = 256 * 16;
  return (int)blocks;
}

// Launch shape of the last-axis kernels: threads along the channel units, blockIdx.y
// along rows; about 64 Ki workgroups (a sweep, as for the per-tensor kernels) of at
// least 4 rows each so the per-channel parameters in registers are reused.
struct LastAxisPlan {
  int bx, by, gx, gy, rows_per_block;
};
inline LastAxisPlan plan_last_axis(int64_t rows, int units) {
  LastAxisPlan p;
  if (units >= kThreads) {
    p.bx = kThreads;
  } else {   // few channels: the next power of two, the rest of the workgroup goes to rows
    p.bx = 1;
    while (p.bx < units) p.bx *= 2;
  }
  p.by = kThreads / p.bx;
  p.gx = (int)dq8::ceil_div(units, p.bx);
  // each thread walks at least four of its rows; rows_per_block is a multiple of by
  int64_t rpb = dq8::ceil_div(rows * p.gx, 65536);
  if (rpb < 4 * p.by) rpb = 4 * p.by;
  rpb = dq8::ceil_div(rpb, p.by) * p.by;
  if (dq8::ceil_div(rows, rpb) > 65535) rpb = dq8::ceil_div(dq8::ceil_div(rows, 65535), p.by) * p.by;
  p.rows_per_block = (int)rpb;
  p.gy = (int)dq8::ceil_div(rows, rpb);
  return p;
}

// one thread per unit, the whole tensor in one sweep
inline unsigned sweep_grid(int64_t units) {
  int64_t blocks = dq8::ceil_div(units, (int64_t)kThreads);
  if (blocks < 1) blocks = 1;
  if (blocks > (1LL << 22)) blocks = 1LL << 22;
  return (unsigned)blocks;
}

}  // namespace elementwise
}  // namespace dq8
