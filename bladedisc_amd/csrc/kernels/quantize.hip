// quantize / dequantize for gfx950: bandwidth-bound, 5 bytes of HBM traffic per
// element.  Semantics follow the reference's runtime decomposition of
// mhlo_disc.quantize / mhlo_disc.dequantize
// (tao_compiler/mlir/disc/transforms/disc_lower_quantize_and_dequantize.cc:77-94,
// 131-136): every step is a separately rounded binary32 operation and the
// division is a true IEEE division, so this file is compiled with
// -ffp-contract=off.
//
// Three access patterns, all without per-element integer division:
//   per tensor            1-D grid-stride over float4 / packed-4 elements
//   per channel, inner==1 (channel is the last axis) 2-D tiles [rows, 4*threads];
//                         each thread keeps its four scales / zero points in
//                         registers while it walks down the rows
//   per channel, inner%4==0 one (outer, channel) row per blockIdx.y
// Anything else (odd sizes, unaligned pointers) takes the scalar kernel.
#include <algorithm>

#include <cstdlib>
#include "dq8_common.h"
#include "disc_q8.h"
#include "q8_elementwise.h"

#pragma clang fp contract(off)

namespace {

using namespace dq8::elementwise;

// Four values quantized with one divisor (or one per component) through its reciprocal: the
// quotients are the bits of x / s (div4_by_constant), so the result is quant_one's; with
// half-to-even rounding, clamping, rounding and byte packing are the epilogue's v_med3 + SDWA
// add.  About 7 vector instructions per element instead of 19 -- with the true division quantize
// was as close to the VALU's limit as to the memory's.
template <int ROUND>
__device__ __forceinline__ uint32_t finish4_quotients(const float4& t, float lo, float hi) {
  if (ROUND == 1) return quant4_pack_rne(t, lo, hi);
  return pack4(quant_from_quotient<ROUND>(t.x, lo, hi), quant_from_quotient<ROUND>(t.y, lo, hi),
               quant_from_quotient<ROUND>(t.z, lo, hi), quant_from_quotient<ROUND>(t.w, lo, hi));
}
template <int ROUND>
__device__ __forceinline__ uint32_t quant4_by_constant(const float4& v, float s, float y, float z,
                                                       float lo, float hi) {
  const float4 q = div4_by_constant(v, s, y);
  return finish4_quotients<ROUND>(make_float4(q.x + z, q.y + z, q.z + z, q.w + z), lo, hi);
}
template <int ROUND>
__device__ __forceinline__ uint32_t quant4_by_constants(const float4& v, const float4& s,
                                                        const float4& y, const float4& z,
                                                        float lo, float hi) {
  const float4 q = div4_by_constants(v, s, y);
  return finish4_quotients<ROUND>(make_float4(q.x + z.x, q.y + z.y, q.z + z.z, q.w + z.w), lo, hi);
}

// ---------------------------------------------------------------- per tensor
// One unit per thread and a grid that covers the tensor in one sweep (the loop only
// runs again beyond 2^30 units): on this part a linear sweep by many small workgroups
// reaches more of the HBM bandwidth than fewer workgroups that each keep several
// far-apart streams in flight (measured on 1 GiB of f32: 6.2 TB/s against 4.7-5.2).
template <int ROUND>
__global__ void __launch_bounds__(kThreads)
quantize_tensor_v4(const float4* __restrict__ x, uint32_t* __restrict__ out,
                   int64_t n4, const float* __restrict__ scale,
                   const int32_t* __restrict__ zp, float lo, float hi) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n4) return;
  // The data load goes out first: a wave has one load to make, and behind the scalar loads of
  // the parameters and the reciprocal it would start a cache miss later.
  float4 v = x[i];
  __builtin_amdgcn_sched_barrier(0);
  const float s = scale[0];
  const float z = (float)zp[0];
  const float y = 1.0f / s;
  const bool fast = divisor_in_fast_range(s);
  for (;;) {
    out[i] = fast ? quant4_by_constant<ROUND>(v, s, y, z, lo, hi)
                  : pack4(quant_one<ROUND>(v.x, s, z, lo, hi), quant_one<ROUND>(v.y, s, z, lo, hi),
                          quant_one<ROUND>(v.z, s, z, lo, hi), quant_one<ROUND>(v.w, s, z, lo, hi));
    i += stride;
    if (i >= n4) break;
    v = x[i];
  }
}

template <bool SIGNED>
__device__ __forceinline__ float4 dequant_word(uint32_t w, int z, float s) {
  const int4 b = unpack4<SIGNED>(w);
  return make_float4((float)(b.x - z) * s, (float)(b.y - z) * s, (float)(b.z - z) * s,
                     (float)(b.w - z) * s);
}

template <bool SIGNED>
__device__ __forceinline__ float4 dequant_word4(uint32_t w, const int4& z, const float4& s) {
  const int4 b = unpack4<SIGNED>(w);
  return make_float4((float)(b.x - z.x) * s.x, (float)(b.y - z.y) * s.y,
                     (float)(b.z - z.z) * s.z, (float)(b.w - z.w) * s.w);
}

// Two 4-byte words in, two 16-byte stores out per thread, one sweep.  A workgroup covers 512
// consecutive words and a thread takes words t and t + 256 of them, so that every load and
// store instruction of a wave covers one contiguous span (64 x 16 bytes per store).  With the
// two words of a thread next to each other (one 8-byte load, stores 32 bytes apart between
// neighbouring lanes) tensors that fit the last-level cache ran a quarter slower:
// [4096,768] 5.35 -> 4.3 us, [32,56,56,64] 8.1 -> 6.1 us, [65536,4096] 221 -> 210 us.
// The f32 results leave with the streaming hint (every store instruction is a whole kilobyte):
// [4096,768] 4.37 -> 3.35 us, [32,56,56,64] 6.3 -> 5.1 us, [65536,4096] 216 -> 187 us, which
// is 7.2 TB/s; the same hint on the loads made every size slower, and on quantize's stores (a
// fifth of its traffic) it helped some sizes and hurt others, so neither is used.
template <bool SIGNED>
__global__ void __launch_bounds__(kThreads)
dequantize_tensor_v4x2(const uint32_t* __restrict__ q, float4* __restrict__ out,
                       int64_t n4, const float* __restrict__ scale,
                       const int32_t* __restrict__ zp) {
  const float s = scale[0];
  const int z = zp[0];
  const int64_t stride = (int64_t)gridDim.x * (2 * kThreads);
  for (int64_t i = (int64_t)blockIdx.x * (2 * kThreads) + threadIdx.x; i < n4; i += stride) {
    const bool two = i + kThreads < n4;
    const uint32_t w0 = q[i];
    const uint32_t w1 = two ? q[i + kThreads] : 0u;
    dq8::st_stream(&out[i], dequant_word<SIGNED>(w0, z, s));
    if (two) dq8::st_stream(&out[i + kThreads], dequant_word<SIGNED>(w1, z, s));
  }
}

// ------------------------------------------- per channel, channel = last axis
// x: [rows, nch], nch % 4 == 0.  threadIdx.x / blockIdx.x tile channels (4 per thread),
// threadIdx.y / blockIdx.y tile rows: each block walks rows_per_block rows, blockDim.y at
// a time (tensors with few channels put several rows side by side in one workgroup).
template <int ROUND>
__global__ void __launch_bounds__(kThreads)
quantize_lastaxis_v4(const float4* __restrict__ x, uint32_t* __restrict__ out,
                     int64_t rows, int nch4, int rows_per_block,
                     const float4* __restrict__ scale,
                     const int4* __restrict__ zp, float lo, float hi) {
  const int c4 = blockIdx.x * blockDim.x + threadIdx.x;
  if (c4 >= nch4) return;
  const float4 s = scale[c4];
  const int4 zi = zp[c4];
  const float4 z = make_float4((float)zi.x, (float)zi.y, (float)zi.z, (float)zi.w);
  const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end = r_begin + rows_per_block < rows ? r_begin + rows_per_block : rows;
  const int64_t step = blockDim.y;               // rows between two rows of this thread
  const int64_t hop = step * nch4;               // the same in units
  int64_t r = r_begin + threadIdx.y;
  const float4* px = x + r * nch4 + c4;
  uint32_t* po = out + r * nch4 + c4;
  const float4 y = make_float4(1.0f / s.x, 1.0f / s.y, 1.0f / s.z, 1.0f / s.w);
  const bool fast = divisor_in_fast_range(s.x) && divisor_in_fast_range(s.y) &&
                    divisor_in_fast_range(s.z) && divisor_in_fast_range(s.w);
  auto one = [&](const float4& v) {
    if (fast) return quant4_by_constants<ROUND>(v, s, y, z, lo, hi);
    return pack4(quant_one<ROUND>(v.x, s.x, z.x, lo, hi), quant_one<ROUND>(v.y, s.y, z.y, lo, hi),
                 quant_one<ROUND>(v.z, s.z, z.z, lo, hi), quant_one<ROUND>(v.w, s.w, z.w, lo, hi));
  };
  for (; r + 3 * step < r_end; r += 4 * step, px += 4 * hop, po += 4 * hop) {
    const float4 v0 = px[0], v1 = px[hop], v2 = px[2 * hop], v3 = px[3 * hop];
    dq8::st_stream(&po[0], one(v0));
    dq8::st_stream(&po[hop], one(v1));
    dq8::st_stream(&po[2 * hop], one(v2));
    dq8::st_stream(&po[3 * hop], one(v3));
  }
  for (; r < r_end; r += step, px += hop, po += hop) dq8::st_stream(&po[0], one(px[0]));
}

template <bool SIGNED>
__global__ void __launch_bounds__(kThreads)
dequantize_lastaxis_v4(const uint32_t* __restrict__ q, float4* __restrict__ out,
                       int64_t rows, int nch4, int rows_per_block,
                       const float4* __restrict__ scale,
                       const int4* __restrict__ zp) {
  const int c4 = blockIdx.x * blockDim.x + threadIdx.x;
  if (c4 >= nch4) return;
  const float4 s = scale[c4];
  const int4 z = zp[c4];
  const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end = r_begin + rows_per_block < rows ? r_begin + rows_per_block : rows;
  const int64_t step = blockDim.y;
  const int64_t hop = step * nch4;
  int64_t r = r_begin + threadIdx.y;
  const uint32_t* pq = q + r * nch4 + c4;
  float4* po = out + r * nch4 + c4;
  for (; r + 3 * step < r_end; r += 4 * step, pq += 4 * hop, po += 4 * hop) {
    const uint32_t w0 = pq[0], w1 = pq[hop], w2 = pq[2 * hop], w3 = pq[3 * hop];
    dq8::st_stream(&po[0], dequant_word4<SIGNED>(w0, z, s));
    dq8::st_stream(&po[hop], dequant_word4<SIGNED>(w1, z, s));
    dq8::st_stream(&po[2 * hop], dequant_word4<SIGNED>(w2, z, s));
    dq8::st_stream(&po[3 * hop], dequant_word4<SIGNED>(w3, z, s));
  }
  for (; r < r_end; r += step, pq += hop, po += hop)
    dq8::st_stream(&po[0], dequant_word4<SIGNED>(pq[0], z, s));
}

// ------------------------------------- per channel, inner % 4 == 0 (any axis)
// One (outer, channel) row of `inner` contiguous elements per blockIdx.y; one unit per
// thread.  The row index is uniform over the workgroup and stays in 32 bits.
template <int ROUND>
__global__ void __launch_bounds__(kThreads)
quantize_rows_v4(const float4* __restrict__ x, uint32_t* __restrict__ out,
                 unsigned rows, int64_t inner4, unsigned nch,
                 const float* __restrict__ scale,
                 const int32_t* __restrict__ zp, float lo, float hi) {
  const unsigned row = blockIdx.y + blockIdx.z * gridDim.y;
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (row >= rows || i >= inner4) return;
  const float4 v = x[(int64_t)row * inner4 + i];
  // The row's parameters stay scalar (the division is cheaper with a uniform divisor)
  // but are fetched after the data load has been issued: a scalar load ahead of it
  // would be waited for, a cold miss per row, before the data load starts.
  __builtin_amdgcn_sched_barrier(0);
  const unsigned c = row % nch;
  const float s = scale[c];
  const float z = (float)zp[c];
  out[(int64_t)row * inner4 + i] =
      divisor_in_fast_range(s)
          ? quant4_by_constant<ROUND>(v, s, 1.0f / s, z, lo, hi)
          : pack4(quant_one<ROUND>(v.x, s, z, lo, hi), quant_one<ROUND>(v.y, s, z, lo, hi),
                  quant_one<ROUND>(v.z, s, z, lo, hi), quant_one<ROUND>(v.w, s, z, lo, hi));
}

// One (outer, channel) row of `inner_words` 4-byte words per blockIdx.y; UNIT words per thread,
// kThreads apart, so that every load and store instruction of a wave is one contiguous span
// (UNIT = 1: 4 bytes in, one 16-byte store; UNIT = 2: two of each).
template <bool SIGNED, int UNIT>
__global__ void __launch_bounds__(kThreads)
dequantize_rows(const uint32_t* __restrict__ q, float4* __restrict__ out,
                unsigned rows, int64_t inner_words, unsigned nch,
                const float* __restrict__ scale, const int32_t* __restrict__ zp) {
  const unsigned row = blockIdx.y + blockIdx.z * gridDim.y;
  if (row >= rows) return;
  const unsigned c = row % nch + opaque_zero();
  const float s = scale[c];
  const int z = zp[c];
  const uint32_t* pq = q + (int64_t)row * inner_words;
  float4* po = out + (int64_t)row * inner_words;
  for (int64_t i = (int64_t)blockIdx.x * (UNIT * kThreads) + threadIdx.x; i < inner_words;
       i += (int64_t)gridDim.x * (UNIT * kThreads)) {
    if (UNIT == 2) {
      const bool two = i + kThreads < inner_words;
      const uint32_t w0 = pq[i];
      const uint32_t w1 = two ? pq[i + kThreads] : 0u;
      dq8::st_stream(&po[i], dequant_word<SIGNED>(w0, z, s));
      if (two) dq8::st_stream(&po[i + kThreads], dequant_word<SIGNED>(w1, z, s));
    } else {
      dq8::st_stream(&po[i], dequant_word<SIGNED>(pq[i], z, s));
    }
  }
}

// ------------------------------------------------------------------ fake quant
// quantize followed by dequantize without the 8-bit tensor in between: f32 in, f32 out,
// the two functions' arithmetic unchanged (the integer result is subtracted from the zero
// point as an integer, as dequantize does).
template <int ROUND>
__device__ __forceinline__ float fake_one(float x, float s, int zi, float lo, float hi) {
  const int q = quant_one<ROUND>(x, s, (float)zi, lo, hi);
  return (float)(q - zi) * s;
}

// fake_one on four values with one divisor through its reciprocal (the quotient's bits are those
// of x / s, see div4_by_constant)
template <int ROUND>
__device__ __forceinline__ float4 fake4_by_constant(const float4& v, float s, float y, int zi,
                                                    float lo, float hi) {
  const float4 q = div4_by_constant(v, s, y);
  const float z = (float)zi;
  auto one = [&](float t0) {
    const int qi = quant_from_quotient<ROUND>(t0 + z, lo, hi);
    return (float)(qi - zi) * s;
  };
  return make_float4(one(q.x), one(q.y), one(q.z), one(q.w));
}

template <int ROUND>
__global__ void __launch_bounds__(kThreads)
fake_quant_tensor_v4(const float4* __restrict__ x, float4* __restrict__ out, int64_t n4,
                     const float* __restrict__ scale, const int32_t* __restrict__ zp, float lo,
                     float hi) {
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n4) return;
  float4 v = x[i];                        // (the data load first, as in quantize_tensor_v4)
  __builtin_amdgcn_sched_barrier(0);
  const float s = scale[0];
  const int z = zp[0];
  const float y = 1.0f / s;
  const bool fast = divisor_in_fast_range(s);
  for (;;) {
    dq8::st_stream(&out[i],
                   fast ? fake4_by_constant<ROUND>(v, s, y, z, lo, hi)
                        : make_float4(fake_one<ROUND>(v.x, s, z, lo, hi), fake_one<ROUND>(v.y, s, z, lo, hi),
                                      fake_one<ROUND>(v.z, s, z, lo, hi), fake_one<ROUND>(v.w, s, z, lo, hi)));
    i += stride;
    if (i >= n4) break;
    v = x[i];
  }
}

template <int ROUND>
__global__ void __launch_bounds__(kThreads)
fake_quant_lastaxis_v4(const float4* __restrict__ x, float4* __restrict__ out, int64_t rows,
                       int nch4, int rows_per_block, const float4* __restrict__ scale,
                       const int4* __restrict__ zp, float lo, float hi) {
  const int c4 = blockIdx.x * blockDim.x + threadIdx.x;
  if (c4 >= nch4) return;
  const float4 s = scale[c4];
  const int4 z = zp[c4];
  const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end = r_begin + rows_per_block < rows ? r_begin + rows_per_block : rows;
  const int64_t step = blockDim.y;
  const int64_t hop = step * nch4;
  int64_t r = r_begin + threadIdx.y;
  const float4* px = x + r * nch4 + c4;
  float4* po = out + r * nch4 + c4;
  auto one = [&](const float4& v) {
    return make_float4(fake_one<ROUND>(v.x, s.x, z.x, lo, hi), fake_one<ROUND>(v.y, s.y, z.y, lo, hi),
                       fake_one<ROUND>(v.z, s.z, z.z, lo, hi), fake_one<ROUND>(v.w, s.w, z.w, lo, hi));
  };
  for (; r + 3 * step < r_end; r += 4 * step, px += 4 * hop, po += 4 * hop) {
    const float4 v0 = px[0], v1 = px[hop], v2 = px[2 * hop], v3 = px[3 * hop];
    dq8::st_stream(&po[0], one(v0));
    dq8::st_stream(&po[hop], one(v1));
    dq8::st_stream(&po[2 * hop], one(v2));
    dq8::st_stream(&po[3 * hop], one(v3));
  }
  for (; r < r_end; r += step, px += hop, po += hop) dq8::st_stream(&po[0], one(px[0]));
}

template <int ROUND>
__global__ void __launch_bounds__(kThreads)
fake_quant_rows_v4(const float4* __restrict__ x, float4* __restrict__ out, unsigned rows,
                   int64_t inner4, unsigned nch, const float* __restrict__ scale,
                   const int32_t* __restrict__ zp, float lo, float hi) {
  const unsigned row = blockIdx.y + blockIdx.z * gridDim.y;
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (row >= rows || i >= inner4) return;
  const float4 v = x[(int64_t)row * inner4 + i];
  __builtin_amdgcn_sched_barrier(0);   // parameters after the data load, as in quantize_rows_v4
  const unsigned c = row % nch;
  const float s = scale[c];
  const int z = zp[c];
  dq8::st_stream(&out[(int64_t)row * inner4 + i],
                 make_float4(fake_one<ROUND>(v.x, s, z, lo, hi), fake_one<ROUND>(v.y, s, z, lo, hi),
                             fake_one<ROUND>(v.z, s, z, lo, hi), fake_one<ROUND>(v.w, s, z, lo, hi)));
}

template <int ROUND>
__global__ void __launch_bounds__(kThreads)
fake_quant_scalar(const float* __restrict__ x, float* __restrict__ out, int64_t begin, int64_t n,
                  int64_t nch, int64_t inner, int per_channel, const float* __restrict__ scale,
                  const int32_t* __restrict__ zp, float lo, float hi) {
  for (int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kThreads) {
    const int64_t c = per_channel ? (i / inner) % nch : 0;
    out[i] = fake_one<ROUND>(x[i], scale[c], zp[c], lo, hi);
  }
}

// ------------------------------------------------------------ scalar fallback
template <int ROUND>
__global__ void __launch_bounds__(kThreads)
quantize_scalar(const float* __restrict__ x, uint8_t* __restrict__ out,
                int64_t begin, int64_t n, int64_t nch, int64_t inner,
                int per_channel, const float* __restrict__ scale,
                const int32_t* __restrict__ zp, float lo, float hi) {
  for (int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kThreads) {
    int64_t c = per_channel ? (i / inner) % nch : 0;
    out[i] = (uint8_t)(quant_one<ROUND>(x[i], scale[c], (float)zp[c], lo, hi) & 0xff);
  }
}

__global__ void __launch_bounds__(kThreads)
dequantize_scalar(const uint8_t* __restrict__ q, float* __restrict__ out,
                  int64_t begin, int64_t n, int64_t nch, int64_t inner,
                  int per_channel, const float* __restrict__ scale,
                  const int32_t* __restrict__ zp, int is_signed) {
  for (int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kThreads) {
    int64_t c = per_channel ? (i / inner) % nch : 0;
    int v = is_signed ? (int)(int8_t)q[i] : (int)q[i];
    out[i] = (float)(v - zp[c]) * scale[c];
  }
}

// ------------------------------------------------- wide outputs, f16 inputs
// 16- and 32-bit quantized types and half-precision inputs: one element per thread, the same
// separately rounded f32 steps.  The conversion of the clamped f32 value saturates: the f32
// images of 2^31 - 1 and 2^32 - 1 are 2^31 and 2^32, one past the integer range.
template <typename QT>
__device__ __forceinline__ QT convert_clamped(float t) {
  return (QT)(int)t;
}
template <>
__device__ __forceinline__ int32_t convert_clamped<int32_t>(float t) {
  return t >= 2147483648.0f ? INT32_MAX : (int32_t)t;
}
template <>
__device__ __forceinline__ uint32_t convert_clamped<uint32_t>(float t) {
  return t >= 4294967296.0f ? UINT32_MAX : (t <= 0.0f ? 0u : (uint32_t)t);
}
template <>
__device__ __forceinline__ uint16_t convert_clamped<uint16_t>(float t) {
  return (uint16_t)(unsigned)t;
}

template <typename XT, typename QT, int ROUND>
__global__ void __launch_bounds__(kThreads)
quantize_wide(const XT* __restrict__ x, QT* __restrict__ out, int64_t n, int64_t nch,
              int64_t inner, int per_channel, const float* __restrict__ scale,
              const int32_t* __restrict__ zp, float lo, float hi) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kThreads) {
    const int64_t c = per_channel ? (i / inner) % nch : 0;
    const float t0 = (float)x[i] / scale[c];
    const float t1 = t0 + (float)zp[c];
    const float t2 = ROUND == DQ8_ROUND_HALF_TO_EVEN ? rintf(t1) : roundf(t1);
    out[i] = convert_clamped<QT>(fminf(fmaxf(t2, lo), hi));
  }
}

template <typename QT>
__global__ void __launch_bounds__(kThreads)
dequantize_wide(const QT* __restrict__ q, float* __restrict__ out, int64_t n, int64_t nch,
                int64_t inner, int per_channel, const float* __restrict__ scale,
                const int32_t* __restrict__ zp) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kThreads) {
    const int64_t c = per_channel ? (i / inner) % nch : 0;
    // the input is converted to the zero point's type (i32) before the subtraction
    out[i] = (float)((int32_t)q[i] - zp[c]) * scale[c];
  }
}

template <typename XT, typename QT>
void launch_quantize_wide(bool rne, const void* x, void* out, int64_t n, int64_t nch,
                          int64_t inner, int per_channel, const float* scale, const int32_t* zp,
                          float lo, float hi, hipStream_t st) {
  const dim3 grid(grid_for(n, 1)), block(kThreads);
  if (rne)
    hipLaunchKernelGGL((quantize_wide<XT, QT, DQ8_ROUND_HALF_TO_EVEN>), grid, block, 0, st,
                       (const XT*)x, (QT*)out, n, nch, inner, per_channel, scale, zp, lo, hi);
  else
    hipLaunchKernelGGL((quantize_wide<XT, QT, DQ8_ROUND_HALF_AWAY_FROM_ZERO>), grid, block, 0, st,
                       (const XT*)x, (QT*)out, n, nch, inner, per_channel, scale, zp, lo, hi);
}

template <typename XT>
bool launch_quantize_kind(int out_kind, bool rne, const void* x, void* out, int64_t n,
                          int64_t nch, int64_t inner, int per_channel, const float* scale,
                          const int32_t* zp, float lo, float hi, hipStream_t st) {
#define DQ8_WIDE_CASE(KIND, QT)                                                              \
  case KIND:                                                                                 \
    launch_quantize_wide<XT, QT>(rne, x, out, n, nch, inner, per_channel, scale, zp, lo, hi, \
                                 st);                                                        \
    return true;
  switch (out_kind) {
    DQ8_WIDE_CASE(DQ8_I8, int8_t)
    DQ8_WIDE_CASE(DQ8_U8, uint8_t)
    DQ8_WIDE_CASE(DQ8_I16, int16_t)
    DQ8_WIDE_CASE(DQ8_U16, uint16_t)
    DQ8_WIDE_CASE(DQ8_I32, int32_t)
    DQ8_WIDE_CASE(DQ8_U32, uint32_t)
  }
#undef DQ8_WIDE_CASE
  return false;
}

}  // namespace

extern "C" int dq8_quantize(const float* x, void* out, int out_kind,
                            int64_t outer, int64_t nch, int64_t inner,
                            const float* scale, const int32_t* zp, int64_t n_q,
                            int32_t qmin, int32_t qmax, int round_mode,
                            void* stream) {
  dq8::clear_error();
  DQ8_REQUIRE(outer >= 0 && nch >= 0 && inner >= 0, "dq8_quantize: negative size");
  DQ8_REQUIRE(out_kind == DQ8_I8 || out_kind == DQ8_U8,
              "dq8_quantize: out_kind must be DQ8_I8 or DQ8_U8");
  DQ8_REQUIRE(round_mode == DQ8_ROUND_HALF_TO_EVEN ||
                  round_mode == DQ8_ROUND_HALF_AWAY_FROM_ZERO,
              "dq8_quantize: unknown round_mode");
  DQ8_REQUIRE(n_q == 1 || n_q == nch, "dq8_quantize: n_q must be 1 or nch");
  const int lim_lo = out_kind == DQ8_I8 ? -128 : 0;
  const int lim_hi = out_kind == DQ8_I8 ? 127 : 255;
  DQ8_REQUIRE(qmin <= qmax && qmin >= lim_lo && qmax <= lim_hi,
              "dq8_quantize: quant_min/quant_max outside the output type");
  const int64_t n = outer * nch * inner;
  if (n == 0) return 0;
  DQ8_REQUIRE(x && out && scale && zp, "dq8_quantize: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const float lo = (float)qmin, hi = (float)qmax;
  const bool per_channel = n_q > 1;
  const bool vec_ok = dq8::aligned(x, 16) && dq8::aligned(out, 4);
  const bool rne = round_mode == DQ8_ROUND_HALF_TO_EVEN;
  // (the kernels divide through the reciprocal, 7 vector instructions per element instead of 19:
  // [4096,768] 3.85 -> 3.3 us, [32,56,56,64] 5.7 -> 4.5 us, [65536,4096] 222-226 -> 216 us)

#define LAUNCH_RND(kernel, grid, block, ...)                                        \
  do {                                                                              \
    if (rne)                                                                        \
      hipLaunchKernelGGL((kernel<DQ8_ROUND_HALF_TO_EVEN>), grid, block, 0, st,      \
                         __VA_ARGS__);                                              \
    else                                                                            \
      hipLaunchKernelGGL((kernel<DQ8_ROUND_HALF_AWAY_FROM_ZERO>), grid, block, 0,   \
                         st, __VA_ARGS__);                                          \
  } while (0)

  if (!per_channel) {
    const int64_t n4 = vec_ok ? n / 4 : 0;
    if (n4 > 0)
      LAUNCH_RND(quantize_tensor_v4, dim3(sweep_grid(n4)), dim3(kThreads),
                 (const float4*)x, (uint32_t*)out, n4, scale, zp, lo, hi);
    if (n4 * 4 < n)
      LAUNCH_RND(quantize_scalar, dim3(grid_for(n - n4 * 4, 1)), dim3(kThreads), x,
                 (uint8_t*)out, n4 * 4, n, (int64_t)1, (int64_t)1, 0, scale, zp, lo, hi);
  } else if (vec_ok && inner == 1 && nch % 4 == 0 && nch / 4 < (1 << 30) &&
             dq8::aligned(scale, 16) && dq8::aligned(zp, 16)) {
    const int nch4 = (int)(nch / 4);
    const LastAxisPlan lp = plan_last_axis(outer, nch4);
    LAUNCH_RND(quantize_lastaxis_v4, dim3(lp.gx, lp.gy), dim3(lp.bx, lp.by), (const float4*)x,
               (uint32_t*)out, outer, nch4, lp.rows_per_block, (const float4*)scale,
               (const int4*)zp, lo, hi);
  } else if (vec_ok && inner % 4 == 0 && outer * nch < (1LL << 31)) {
    const int64_t rows = outer * nch;
    const int64_t inner4 = inner / 4;
    DQ8_REQUIRE(inner4 < (1LL << 38), "dq8_quantize: rows too long for one launch");
    unsigned gx = (unsigned)dq8::ceil_div(inner4, kThreads);
    int gy = (int)std::min<int64_t>(rows, 32768);
    int64_t gz = dq8::ceil_div(rows, gy);
    DQ8_REQUIRE(gz <= 65535, "dq8_quantize: too many rows for one launch");
    LAUNCH_RND(quantize_rows_v4, dim3(gx, gy, (unsigned)gz), dim3(kThreads),
               (const float4*)x, (uint32_t*)out, (unsigned)rows, inner4, (unsigned)nch, scale,
               zp, lo, hi);
  } else {
    LAUNCH_RND(quantize_scalar, dim3(grid_for(n, 1)), dim3(kThreads), x,
               (uint8_t*)out, (int64_t)0, n, nch, inner, 1, scale, zp, lo, hi);
  }
#undef LAUNCH_RND
  return dq8::check_hip(hipGetLastError(), "dq8_quantize launch");
}

extern "C" int dq8_dequantize(const void* q, int in_kind, float* out,
                              int64_t outer, int64_t nch, int64_t inner,
                              const float* scale, const int32_t* zp,
                              int64_t n_q, void* stream) {
  dq8::clear_error();
  DQ8_REQUIRE(outer >= 0 && nch >= 0 && inner >= 0, "dq8_dequantize: negative size");
  DQ8_REQUIRE(in_kind == DQ8_I8 || in_kind == DQ8_U8,
              "dq8_dequantize: in_kind must be DQ8_I8 or DQ8_U8");
  DQ8_REQUIRE(n_q == 1 || n_q == nch, "dq8_dequantize: n_q must be 1 or nch");
  const int64_t n = outer * nch * inner;
  if (n == 0) return 0;
  DQ8_REQUIRE(q && out && scale && zp, "dq8_dequantize: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const int is_signed = in_kind == DQ8_I8;
  const bool per_channel = n_q > 1;
  const bool vec_ok = dq8::aligned(q, 4) && dq8::aligned(out, 16);

  if (!per_channel) {
    const int64_t n4 = vec_ok ? n / 4 : 0;
    if (n4 > 0) {
      auto k = is_signed ? dequantize_tensor_v4x2<true> : dequantize_tensor_v4x2<false>;
      hipLaunchKernelGGL(k, dim3(sweep_grid(dq8::ceil_div(n4, 2))), dim3(kThreads), 0, st,
                         (const uint32_t*)q, (float4*)out, n4, scale, zp);
    }
    if (n4 * 4 < n)
      hipLaunchKernelGGL(dequantize_scalar, dim3(grid_for(n - n4 * 4, 1)),
                         dim3(kThreads), 0, st, (const uint8_t*)q, out, n4 * 4, n,
                         (int64_t)1, (int64_t)1, 0, scale, zp, is_signed);
  } else if (vec_ok && inner == 1 && nch % 4 == 0 && nch / 4 < (1 << 30) &&
             dq8::aligned(scale, 16) && dq8::aligned(zp, 16)) {
    const int nch4 = (int)(nch / 4);
    const LastAxisPlan lp = plan_last_axis(outer, nch4);
    auto k = is_signed ? dequantize_lastaxis_v4<true> : dequantize_lastaxis_v4<false>;
    hipLaunchKernelGGL(k, dim3(lp.gx, lp.gy), dim3(lp.bx, lp.by), 0, st, (const uint32_t*)q,
                       (float4*)out, outer, nch4, lp.rows_per_block, (const float4*)scale,
                       (const int4*)zp);
  } else if (vec_ok && inner % 4 == 0 && outer * nch < (1LL << 31)) {
    const int64_t rows = outer * nch;
    const bool v8 = inner >= 2048;     // two words per thread once a row is several workgroups
    const int64_t units = inner / 4;
    int gx = (int)std::min<int64_t>(dq8::ceil_div(units, kThreads * (v8 ? 2 : 1)), 65536);
    int gy = (int)std::min<int64_t>(rows, 32768);
    int64_t gz = dq8::ceil_div(rows, gy);
    DQ8_REQUIRE(gz <= 65535, "dq8_dequantize: too many rows for one launch");
    auto k = v8 ? (is_signed ? dequantize_rows<true, 2> : dequantize_rows<false, 2>)
                : (is_signed ? dequantize_rows<true, 1> : dequantize_rows<false, 1>);
    hipLaunchKernelGGL(k, dim3(gx, gy, (unsigned)gz), dim3(kThreads), 0, st,
                       (const uint32_t*)q, (float4*)out, (unsigned)rows, units, (unsigned)nch,
                       scale, zp);
  } else {
    hipLaunchKernelGGL(dequantize_scalar, dim3(grid_for(n, 1)), dim3(kThreads), 0,
                       st, (const uint8_t*)q, out, (int64_t)0, n, nch, inner, 1,
                       scale, zp, is_signed);
  }
  return dq8::check_hip(hipGetLastError(), "dq8_dequantize launch");
}

extern "C" int dq8_fake_quant(const float* x, float* out, int64_t outer, int64_t nch,
                              int64_t inner, const float* scale, const int32_t* zp, int64_t n_q,
                              int32_t qmin, int32_t qmax, int round_mode, void* stream) {
  dq8::clear_error();
  DQ8_REQUIRE(outer >= 0 && nch >= 0 && inner >= 0, "dq8_fake_quant: negative size");
  DQ8_REQUIRE(round_mode == DQ8_ROUND_HALF_TO_EVEN ||
                  round_mode == DQ8_ROUND_HALF_AWAY_FROM_ZERO,
              "dq8_fake_quant: unknown round_mode");
  DQ8_REQUIRE(n_q == 1 || n_q == nch, "dq8_fake_quant: n_q must be 1 or nch");
  DQ8_REQUIRE(qmin <= qmax && qmin >= -32768 && qmax <= 65535,
              "dq8_fake_quant: quant_min/quant_max outside the 8- and 16-bit ranges");
  const int64_t n = outer * nch * inner;
  if (n == 0) return 0;
  DQ8_REQUIRE(x && out && scale && zp, "dq8_fake_quant: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const float lo = (float)qmin, hi = (float)qmax;
  const bool per_channel = n_q > 1;
  const bool vec_ok = dq8::aligned(x, 16) && dq8::aligned(out, 16);
  const bool rne = round_mode == DQ8_ROUND_HALF_TO_EVEN;

#define LAUNCH_RND(kernel, grid, block, ...)                                        \
  do {                                                                              \
    if (rne)                                                                        \
      hipLaunchKernelGGL((kernel<DQ8_ROUND_HALF_TO_EVEN>), grid, block, 0, st,      \
                         __VA_ARGS__);                                              \
    else                                                                            \
      hipLaunchKernelGGL((kernel<DQ8_ROUND_HALF_AWAY_FROM_ZERO>), grid, block, 0,   \
                         st, __VA_ARGS__);                                          \
  } while (0)

  if (!per_channel) {
    const int64_t n4 = vec_ok ? n / 4 : 0;
    if (n4 > 0)
      LAUNCH_RND(fake_quant_tensor_v4, dim3(sweep_grid(n4)), dim3(kThreads), (const float4*)x,
                 (float4*)out, n4, scale, zp, lo, hi);
    if (n4 * 4 < n)
      LAUNCH_RND(fake_quant_scalar, dim3(grid_for(n - n4 * 4, 1)), dim3(kThreads), x, out,
                 n4 * 4, n, (int64_t)1, (int64_t)1, 0, scale, zp, lo, hi);
  } else if (vec_ok && inner == 1 && nch % 4 == 0 && nch / 4 < (1 << 30) &&
             dq8::aligned(scale, 16) && dq8::aligned(zp, 16)) {
    const int nch4 = (int)(nch / 4);
    const LastAxisPlan lp = plan_last_axis(outer, nch4);
    LAUNCH_RND(fake_quant_lastaxis_v4, dim3(lp.gx, lp.gy), dim3(lp.bx, lp.by), (const float4*)x,
               (float4*)out, outer, nch4, lp.rows_per_block, (const float4*)scale,
               (const int4*)zp, lo, hi);
  } else if (vec_ok && inner % 4 == 0 && outer * nch < (1LL << 31) &&
             inner / 4 < (1LL << 38) && dq8::ceil_div(outer * nch, 32768) <= 65535) {
    const int64_t rows = outer * nch;
    const int64_t inner4 = inner / 4;
    const unsigned gx = (unsigned)dq8::ceil_div(inner4, kThreads);
    const int gy = (int)std::min<int64_t>(rows, 32768);
    const int64_t gz = dq8::ceil_div(rows, gy);
    LAUNCH_RND(fake_quant_rows_v4, dim3(gx, gy, (unsigned)gz), dim3(kThreads), (const float4*)x,
               (float4*)out, (unsigned)rows, inner4, (unsigned)nch, scale, zp, lo, hi);
  } else {
    LAUNCH_RND(fake_quant_scalar, dim3(grid_for(n, 1)), dim3(kThreads), x, out, (int64_t)0, n,
               nch, inner, 1, scale, zp, lo, hi);
  }
#undef LAUNCH_RND
  return dq8::check_hip(hipGetLastError(), "dq8_fake_quant launch");
}

namespace {
bool quant_limits(int kind, int64_t* lo, int64_t* hi) {
  switch (kind) {
    case DQ8_I8: *lo = -128; *hi = 127; return true;
    case DQ8_U8: *lo = 0; *hi = 255; return true;
    case DQ8_I16: *lo = -32768; *hi = 32767; return true;
    case DQ8_U16: *lo = 0; *hi = 65535; return true;
    case DQ8_I32: *lo = INT32_MIN; *hi = INT32_MAX; return true;
    case DQ8_U32: *lo = 0; *hi = UINT32_MAX; return true;
  }
  return false;
}
}  // namespace

extern "C" int dq8_quantize_ex(const void* x, int x_dtype, void* out, int out_kind, int64_t outer,
                               int64_t nch, int64_t inner, const float* scale,
                               const int32_t* zp, int64_t n_q, int64_t qmin, int64_t qmax,
                               int round_mode, void* stream) {
  dq8::clear_error();
  int64_t lim_lo = 0, lim_hi = 0;
  DQ8_REQUIRE(quant_limits(out_kind, &lim_lo, &lim_hi), "dq8_quantize_ex: unknown out_kind");
  DQ8_REQUIRE(x_dtype == DQ8_DTYPE_F32 || x_dtype == DQ8_DTYPE_F16,
              "dq8_quantize_ex: input must be f32 or f16");
  DQ8_REQUIRE(qmin <= qmax && qmin >= lim_lo && qmax <= lim_hi,
              "dq8_quantize_ex: quant_min/quant_max outside the output type");
  // f32 -> 8 bit: the bandwidth-tuned kernels
  if (x_dtype == DQ8_DTYPE_F32 && (out_kind == DQ8_I8 || out_kind == DQ8_U8))
    return dq8_quantize(static_cast<const float*>(x), out, out_kind, outer, nch, inner, scale, zp,
                        n_q, (int32_t)qmin, (int32_t)qmax, round_mode, stream);
  DQ8_REQUIRE(outer >= 0 && nch >= 0 && inner >= 0, "dq8_quantize_ex: negative size");
  DQ8_REQUIRE(round_mode == DQ8_ROUND_HALF_TO_EVEN ||
                  round_mode == DQ8_ROUND_HALF_AWAY_FROM_ZERO,
              "dq8_quantize_ex: unknown round_mode");
  DQ8_REQUIRE(n_q == 1 || n_q == nch, "dq8_quantize_ex: n_q must be 1 or nch");
  const int64_t n = outer * nch * inner;
  if (n == 0) return 0;
  DQ8_REQUIRE(x && out && scale && zp, "dq8_quantize_ex: null pointer");
  const bool rne = round_mode == DQ8_ROUND_HALF_TO_EVEN;
  const float lo = (float)qmin, hi = (float)qmax;
  hipStream_t st = (hipStream_t)stream;
  if (x_dtype == DQ8_DTYPE_F32)
    launch_quantize_kind<float>(out_kind, rne, x, out, n, nch, inner, n_q > 1, scale, zp, lo, hi,
                                st);
  else
    launch_quantize_kind<_Float16>(out_kind, rne, x, out, n, nch, inner, n_q > 1, scale, zp, lo,
                                   hi, st);
  return dq8::check_hip(hipGetLastError(), "dq8_quantize_ex launch");
}

extern "C" int dq8_dequantize_ex(const void* q, int in_kind, float* out, int64_t outer,
                                 int64_t nch, int64_t inner, const float* scale,
                                 const int32_t* zp, int64_t n_q, void* stream) {
  if (in_kind == DQ8_I8 || in_kind == DQ8_U8)
    return dq8_dequantize(q, in_kind, out, outer, nch, inner, scale, zp, n_q, stream);
  dq8::clear_error();
  DQ8_REQUIRE(in_kind >= DQ8_I16 && in_kind <= DQ8_U32, "dq8_dequantize_ex: unknown in_kind");
  DQ8_REQUIRE(outer >= 0 && nch >= 0 && inner >= 0, "dq8_dequantize_ex: negative size");
  DQ8_REQUIRE(n_q == 1 || n_q == nch, "dq8_dequantize_ex: n_q must be 1 or nch");
  const int64_t n = outer * nch * inner;
  if (n == 0) return 0;
  DQ8_REQUIRE(q && out && scale && zp, "dq8_dequantize_ex: null pointer");
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(grid_for(n, 1)), block(kThreads);
  const int pc = n_q > 1;
#define DQ8_WIDE_CASE(QT)                                                                   \
  hipLaunchKernelGGL(dequantize_wide<QT>, grid, block, 0, st, (const QT*)q, out, n, nch, inner, \
                     pc, scale, zp)
  switch (in_kind) {
    case DQ8_I16: DQ8_WIDE_CASE(int16_t); break;
    case DQ8_U16: DQ8_WIDE_CASE(uint16_t); break;
    case DQ8_I32: DQ8_WIDE_CASE(int32_t); break;
    default: DQ8_WIDE_CASE(uint32_t); break;
  }
#undef DQ8_WIDE_CASE
  return dq8::check_hip(hipGetLastError(), "dq8_dequantize_ex launch");
}
