// TensorFlow's QuantizeV2 (modes SCALED and MIN_FIRST) and Dequantize (SCALED) as the
// reference lowers them (tao_compiler/mlir/disc/transforms/lower_tf.cc:307-654): chains of
// elementwise f32 operations over the data and the min / max range operands.  Here the
// range arithmetic runs once per channel in a small kernel that leaves four floats per
// channel in a parameter array, and one bandwidth-bound pass (5 bytes per element) applies
//     q = clamp(round(clamp(x, lo, hi) * m) - b, lowest, highest)
// with the same separately rounded operations the lowering emits (no contraction; the
// data is multiplied by the factor, not divided by its reciprocal).  Rounding is
// tf.Round's, half to even.
//   SCALED    lo / hi = the adjusted range, m = the scale factor, b = 0
//   MIN_FIRST lo / hi = -inf / +inf,        m = (max - min) / 255, b = round(min m) - lowest
// Dequantize multiplies by a per-channel factor, which is dq8_dequantize with a zero point
// of zero; only its range arithmetic is new.
#include <cfloat>
#include <cmath>

#include "dq8_common.h"
#include "disc_q8.h"
#include "q8_elementwise.h"

#pragma clang fp contract(off)

namespace {

using namespace dq8::elementwise;

struct OutLimits {
  float lowest, highest, min_q;   // min_q = lowest + narrow_range
};

// lower_tf.cc:365-393
__device__ __forceinline__ void adjust_range(float mn, float mx, float ensure, float* lo,
                                             float* hi) {
  *lo = fminf(0.f, mn);
  float eps = fmaxf(fmaxf(fabsf(mn), fabsf(mx)), 1.f);
  eps = eps * ensure;
  float h = eps + *lo;
  h = fmaxf(mx, h);
  *hi = fmaxf(0.f, h);
}

// One thread per channel: params[c] = {lo, hi, m, b}; out_min / out_max are the op's second
// and third results.
__global__ void __launch_bounds__(kThreads)
tf_quantize_params(const float* __restrict__ min_range, const float* __restrict__ max_range,
                   int64_t channels, int mode, OutLimits lim, float ensure,
                   float* __restrict__ out_min, float* __restrict__ out_max,
                   float4* __restrict__ params) {
  const int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  float lo, hi;
  adjust_range(min_range[c], max_range[c], ensure, &lo, &hi);
  if (mode == DQ8_TF_MIN_FIRST) {               // lower_tf.cc:415-444
    float rs = hi - lo;
    rs = rs / 255.f;
    float rms = rintf(lo * rs);
    out_min[c] = lo;
    out_max[c] = hi;
    params[c] = make_float4(-INFINITY, INFINITY, rs, rms - lim.lowest);
    return;
  }
  // lower_tf.cc:476-538
  const float adj_lo = lo - (lo == 0.f ? 1.f : 0.f) * 1e-6f;
  float sf_lo = lim.min_q / adj_lo;
  sf_lo = lo * lim.min_q > 0.f ? sf_lo : FLT_MAX;
  const float adj_hi = hi - (hi == 0.f ? 1.f : 0.f) * 1e-6f;
  float sf_hi = lim.highest / adj_hi;
  sf_hi = hi * lim.highest > 0.f ? sf_hi : FLT_MAX;
  const float sf = fminf(sf_lo, sf_hi);
  const float qlo = lim.min_q / sf;
  const float qhi = lim.highest / sf;
  out_min[c] = qlo;
  out_max[c] = qhi;
  params[c] = make_float4(qlo, qhi, sf, 0.f);
}

// lower_tf.cc:629-644: scale[c] = max(min / min_q, max / highest) (signed) or max / highest;
// zp[c] = 0.  Channels are padded to a multiple of four in both arrays.
__global__ void __launch_bounds__(kThreads)
tf_dequantize_params(const float* __restrict__ min_range, const float* __restrict__ max_range,
                     int64_t channels, OutLimits lim, float* __restrict__ scale,
                     int32_t* __restrict__ zp) {
  const int64_t c = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (c >= channels) return;
  float sf = max_range[c] / lim.highest;
  if (lim.lowest != 0.f) sf = fmaxf(min_range[c] / lim.min_q, sf);
  scale[c] = sf;
  zp[c] = 0;
}

__device__ __forceinline__ int tf_quant_one(float x, const float4& p, float lb, float ub) {
  float t = fminf(fmaxf(x, p.x), p.y);   // a NaN takes the lower bound
  t = t * p.z;
  t = rintf(t);
  t = t - p.w;
  t = fminf(fmaxf(t, lb), ub);
  return (int)t;
}

__device__ __forceinline__ uint32_t tf_quant_four(const float4& v, const float4& p, float lb,
                                                  float ub) {
  return pack4(tf_quant_one(v.x, p, lb, ub), tf_quant_one(v.y, p, lb, ub),
               tf_quant_one(v.z, p, lb, ub), tf_quant_one(v.w, p, lb, ub));
}

// per tensor: one float4 per thread, the whole tensor in one sweep
__global__ void __launch_bounds__(kThreads)
tf_quantize_tensor_v4(const float4* __restrict__ x, uint32_t* __restrict__ out, int64_t n4,
                      const float4* __restrict__ params, float lb, float ub) {
  const float4 p = params[0];
  const int64_t stride = (int64_t)gridDim.x * kThreads;
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n4; i += stride)
    out[i] = tf_quant_four(x[i], p, lb, ub);
}

// channel = last axis, channels % 4 == 0: each thread keeps the parameters of its four
// channels in registers while it walks down its rows
__global__ void __launch_bounds__(kThreads)
tf_quantize_lastaxis_v4(const float4* __restrict__ x, uint32_t* __restrict__ out, int64_t rows,
                        int nch4, int rows_per_block, const float4* __restrict__ params,
                        float lb, float ub) {
  const int c4 = blockIdx.x * blockDim.x + threadIdx.x;
  if (c4 >= nch4) return;
  const float4 p0 = params[4 * c4], p1 = params[4 * c4 + 1], p2 = params[4 * c4 + 2],
               p3 = params[4 * c4 + 3];
  const int64_t r_begin = (int64_t)blockIdx.y * rows_per_block;
  const int64_t r_end = r_begin + rows_per_block < rows ? r_begin + rows_per_block : rows;
  const int64_t step = blockDim.y;
  const int64_t hop = step * nch4;
  int64_t r = r_begin + threadIdx.y;
  const float4* px = x + r * nch4 + c4;
  uint32_t* po = out + r * nch4 + c4;
  auto one = [&](const float4& v) {
    return pack4(tf_quant_one(v.x, p0, lb, ub), tf_quant_one(v.y, p1, lb, ub),
                 tf_quant_one(v.z, p2, lb, ub), tf_quant_one(v.w, p3, lb, ub));
  };
  for (; r + 3 * step < r_end; r += 4 * step, px += 4 * hop, po += 4 * hop) {
    const float4 v0 = px[0], v1 = px[hop], v2 = px[2 * hop], v3 = px[3 * hop];
    po[0] = one(v0);
    po[hop] = one(v1);
    po[2 * hop] = one(v2);
    po[3 * hop] = one(v3);
  }
  for (; r < r_end; r += step, px += hop, po += hop) po[0] = one(px[0]);
}

// inner % 4 == 0: one (outer, channel) row per blockIdx.y, one unit per thread
__global__ void __launch_bounds__(kThreads)
tf_quantize_rows_v4(const float4* __restrict__ x, uint32_t* __restrict__ out, unsigned rows,
                    int64_t inner4, unsigned nch, const float4* __restrict__ params, float lb,
                    float ub) {
  const unsigned row = blockIdx.y + blockIdx.z * gridDim.y;
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (row >= rows || i >= inner4) return;
  const float4 v = x[(int64_t)row * inner4 + i];
  const float4 p = params[row % nch + opaque_zero()];
  out[(int64_t)row * inner4 + i] = tf_quant_four(v, p, lb, ub);
}

__global__ void __launch_bounds__(kThreads)
tf_quantize_scalar(const float* __restrict__ x, uint8_t* __restrict__ out, int64_t begin,
                   int64_t n, int64_t nch, int64_t inner, const float4* __restrict__ params,
                   float lb, float ub) {
  for (int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * kThreads) {
    const int64_t c = nch > 1 ? (i / inner) % nch : 0;
    out[i] = (uint8_t)(tf_quant_one(x[i], params[c], lb, ub) & 0xff);
  }
}

int64_t padded4(int64_t channels) { return (channels + 3) / 4 * 4; }

}  // namespace

extern "C" size_t dq8_tf_params_bytes(int64_t channels) {
  if (channels < 1) channels = 1;
  return (size_t)padded4(channels) * 16;
}

extern "C" int dq8_tf_quantize_v2(const float* x, void* out, int out_kind, int64_t outer,
                                  int64_t channels, int64_t inner, const float* min_range,
                                  const float* max_range, int mode, int narrow_range,
                                  float ensure_minimum_range, float* out_min, float* out_max,
                                  void* params, size_t params_bytes, void* stream) {
  dq8::clear_error();
  DQ8_REQUIRE(outer >= 0 && channels >= 0 && inner >= 0, "dq8_tf_quantize_v2: negative size");
  DQ8_REQUIRE(out_kind == DQ8_I8 || out_kind == DQ8_U8,
              "dq8_tf_quantize_v2: out_kind must be DQ8_I8 or DQ8_U8");
  DQ8_REQUIRE(mode == DQ8_TF_SCALED || mode == DQ8_TF_MIN_FIRST,
              "dq8_tf_quantize_v2: mode must be DQ8_TF_SCALED or DQ8_TF_MIN_FIRST");
  DQ8_REQUIRE(mode != DQ8_TF_MIN_FIRST || channels <= 1,
              "dq8_tf_quantize_v2: MIN_FIRST takes scalar ranges");
  const int64_t n = outer * channels * inner;
  if (channels == 0) return 0;
  DQ8_REQUIRE(min_range && max_range && out_min && out_max && params,
              "dq8_tf_quantize_v2: null pointer");
  DQ8_REQUIRE(dq8::aligned(params, 16) && params_bytes >= dq8_tf_params_bytes(channels),
              "dq8_tf_quantize_v2: params must be 16-byte aligned and hold dq8_tf_params_bytes()");
  hipStream_t st = (hipStream_t)stream;
  OutLimits lim;
  lim.lowest = out_kind == DQ8_I8 ? -128.f : 0.f;
  lim.highest = out_kind == DQ8_I8 ? 127.f : 255.f;
  lim.min_q = lim.lowest + (narrow_range ? 1.f : 0.f);
  hipLaunchKernelGGL(tf_quantize_params, dim3((unsigned)dq8::ceil_div(channels, kThreads)),
                     dim3(kThreads), 0, st, min_range, max_range, channels, mode, lim,
                     ensure_minimum_range, out_min, out_max, (float4*)params);
  if (n == 0) return dq8::check_hip(hipGetLastError(), "dq8_tf_quantize_v2 launch");
  DQ8_REQUIRE(x && out, "dq8_tf_quantize_v2: null pointer");
  const float4* p = (const float4*)params;
  const float lb = lim.lowest, ub = lim.highest;
  const bool vec_ok = dq8::aligned(x, 16) && dq8::aligned(out, 4);

  if (channels == 1) {
    const int64_t n4 = vec_ok ? n / 4 : 0;
    if (n4 > 0)
      hipLaunchKernelGGL(tf_quantize_tensor_v4, dim3(sweep_grid(n4)), dim3(kThreads), 0, st,
                         (const float4*)x, (uint32_t*)out, n4, p, lb, ub);
    if (n4 * 4 < n)
      hipLaunchKernelGGL(tf_quantize_scalar, dim3(grid_for(n - n4 * 4, 1)), dim3(kThreads), 0,
                         st, x, (uint8_t*)out, n4 * 4, n, (int64_t)1, (int64_t)1, p, lb, ub);
  } else if (vec_ok && inner == 1 && channels % 4 == 0 && channels / 4 < (1 << 30)) {
    const int nch4 = (int)(channels / 4);
    const LastAxisPlan lp = plan_last_axis(outer, nch4);
    hipLaunchKernelGGL(tf_quantize_lastaxis_v4, dim3(lp.gx, lp.gy), dim3(lp.bx, lp.by), 0, st,
                       (const float4*)x, (uint32_t*)out, outer, nch4, lp.rows_per_block, p, lb,
                       ub);
  } else if (vec_ok && inner % 4 == 0 && outer * channels < (1LL << 31) &&
             inner / 4 < (1LL << 38) && dq8::ceil_div(outer * channels, 32768) <= 65535) {
    const int64_t rows = outer * channels;
    const int64_t inner4 = inner / 4;
    const unsigned gx = (unsigned)dq8::ceil_div(inner4, kThreads);
    const int gy = (int)std::min<int64_t>(rows, 32768);
    const int64_t gz = dq8::ceil_div(rows, gy);
    hipLaunchKernelGGL(tf_quantize_rows_v4, dim3(gx, gy, (unsigned)gz), dim3(kThreads), 0, st,
                       (const float4*)x, (uint32_t*)out, (unsigned)rows, inner4,
                       (unsigned)channels, p, lb, ub);
  } else {
    hipLaunchKernelGGL(tf_quantize_scalar, dim3(grid_for(n, 1)), dim3(kThreads), 0, st, x,
                       (uint8_t*)out, (int64_t)0, n, channels, inner, p, lb, ub);
  }
  return dq8::check_hip(hipGetLastError(), "dq8_tf_quantize_v2 launch");
}

extern "C" int dq8_tf_dequantize(const void* q, int in_kind, float* out, int64_t outer,
                                 int64_t channels, int64_t inner, const float* min_range,
                                 const float* max_range, int narrow_range, void* params,
                                 size_t params_bytes, void* stream) {
  dq8::clear_error();
  DQ8_REQUIRE(outer >= 0 && channels >= 0 && inner >= 0, "dq8_tf_dequantize: negative size");
  DQ8_REQUIRE(in_kind == DQ8_I8 || in_kind == DQ8_U8,
              "dq8_tf_dequantize: in_kind must be DQ8_I8 or DQ8_U8");
  if (outer * channels * inner == 0) return 0;
  DQ8_REQUIRE(q && out && min_range && max_range && params, "dq8_tf_dequantize: null pointer");
  DQ8_REQUIRE(dq8::aligned(params, 16) && params_bytes >= dq8_tf_params_bytes(channels),
              "dq8_tf_dequantize: params must be 16-byte aligned and hold dq8_tf_params_bytes()");
  OutLimits lim;
  lim.lowest = in_kind == DQ8_I8 ? -128.f : 0.f;
  lim.highest = in_kind == DQ8_I8 ? 127.f : 255.f;
  lim.min_q = lim.lowest + (narrow_range ? 1.f : 0.f);
  float* scale = (float*)params;
  int32_t* zp = (int32_t*)params + padded4(channels);
  hipLaunchKernelGGL(tf_dequantize_params, dim3((unsigned)dq8::ceil_div(channels, kThreads)),
                     dim3(kThreads), 0, (hipStream_t)stream, min_range, max_range, channels, lim,
                     scale, zp);
  int rc = dq8::check_hip(hipGetLastError(), "dq8_tf_dequantize launch");
  if (rc) return rc;
  return dq8_dequantize(q, in_kind, out, outer, channels, inner, scale, zp, channels, stream);
}
