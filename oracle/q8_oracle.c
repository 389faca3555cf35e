/*
 * q8_oracle.c -- see q8_oracle.h.  TEST INFRASTRUCTURE ONLY: the checker and the
 * timed CPU baseline; never part of the shipped GPU path.
 *
 * Build with -ffp-contract=off: every float operation below is meant to be a
 * separately rounded IEEE binary32 operation, as in the reference's CPU path.
 */
#include "q8_oracle.h"

#include <fenv.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#if defined(__x86_64__)
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------------ */
/* int32 accumulation                                                        */
/* R: ral/context/common_context_impl_quantization.cc:1219-1234 (m,k,n and   */
/*    the ab/ba format tags selected by tp_a / tp_b)                         */
/* ------------------------------------------------------------------------ */
void q8o_gemm_s32(const int8_t* A, const int8_t* W, int32_t* acc, int64_t M,
                  int64_t N, int64_t K, int tp_a, int tp_b, int32_t zx,
                  int32_t zw) {
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      int32_t s = 0;
      for (int64_t k = 0; k < K; ++k) {
        int32_t a = tp_a ? A[k * M + m] : A[m * K + k];
        int32_t w = tp_b ? W[n * K + k] : W[k * N + n];
        s += (a - zx) * (w - zw);
      }
      acc[m * N + n] = s;
    }
  }
}

static void gemm_nt_rows_plain(const int8_t* A, const int8_t* Wnk, int32_t* acc,
                               int64_t m0, int64_t m1, int64_t N, int64_t K) {
  for (int64_t m = m0; m < m1; ++m) {
    const int8_t* a = A + m * K;
    for (int64_t n = 0; n < N; ++n) {
      const int8_t* w = Wnk + n * K;
      int32_t s = 0;
      for (int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)w[k];
      acc[m * N + n] = s;
    }
  }
}

#if defined(__x86_64__)
/* vpdpbusd multiplies unsigned by signed bytes: feed a+128 and subtract
 * 128*sum_k w[n,k] afterwards (exact in int32 for K*255*128 < 2^31). */
__attribute__((target("avx512f,avx512bw,avx512vl,avx512vnni"))) static void
gemm_nt_rows_vnni(const int8_t* A, const int8_t* Wnk, const int32_t* wsum,
                  int32_t* acc, int64_t m0, int64_t m1, int64_t N, int64_t K) {
  const __m512i flip = _mm512_set1_epi8((char)0x80);
  const int64_t K64 = K & ~(int64_t)63;
  int64_t m = m0;
  for (; m + 4 <= m1; m += 4) {
    const int8_t* a0 = A + (m + 0) * K;
    const int8_t* a1 = A + (m + 1) * K;
    const int8_t* a2 = A + (m + 2) * K;
    const int8_t* a3 = A + (m + 3) * K;
    int64_t n = 0;
    for (; n + 4 <= N; n += 4) {
      __m512i c[16];
      for (int i = 0; i < 16; ++i) c[i] = _mm512_setzero_si512();
      const int8_t* w0 = Wnk + (n + 0) * K;
      const int8_t* w1 = Wnk + (n + 1) * K;
      const int8_t* w2 = Wnk + (n + 2) * K;
      const int8_t* w3 = Wnk + (n + 3) * K;
      for (int64_t k = 0; k < K64; k += 64) {
        __m512i x0 = _mm512_xor_si512(_mm512_loadu_si512(a0 + k), flip);
        __m512i x1 = _mm512_xor_si512(_mm512_loadu_si512(a1 + k), flip);
        __m512i x2 = _mm512_xor_si512(_mm512_loadu_si512(a2 + k), flip);
        __m512i x3 = _mm512_xor_si512(_mm512_loadu_si512(a3 + k), flip);
        __m512i y0 = _mm512_loadu_si512(w0 + k);
        __m512i y1 = _mm512_loadu_si512(w1 + k);
        __m512i y2 = _mm512_loadu_si512(w2 + k);
        __m512i y3 = _mm512_loadu_si512(w3 + k);
        c[0] = _mm512_dpbusd_epi32(c[0], x0, y0);
        c[1] = _mm512_dpbusd_epi32(c[1], x0, y1);
        c[2] = _mm512_dpbusd_epi32(c[2], x0, y2);
        c[3] = _mm512_dpbusd_epi32(c[3], x0, y3);
        c[4] = _mm512_dpbusd_epi32(c[4], x1, y0);
        c[5] = _mm512_dpbusd_epi32(c[5], x1, y1);
        c[6] = _mm512_dpbusd_epi32(c[6], x1, y2);
        c[7] = _mm512_dpbusd_epi32(c[7], x1, y3);
        c[8] = _mm512_dpbusd_epi32(c[8], x2, y0);
        c[9] = _mm512_dpbusd_epi32(c[9], x2, y1);
        c[10] = _mm512_dpbusd_epi32(c[10], x2, y2);
        c[11] = _mm512_dpbusd_epi32(c[11], x2, y3);
        c[12] = _mm512_dpbusd_epi32(c[12], x3, y0);
        c[13] = _mm512_dpbusd_epi32(c[13], x3, y1);
        c[14] = _mm512_dpbusd_epi32(c[14], x3, y2);
        c[15] = _mm512_dpbusd_epi32(c[15], x3, y3);
      }
      const int8_t* ar[4] = {a0, a1, a2, a3};
      const int8_t* wr[4] = {w0, w1, w2, w3};
      for (int i = 0; i < 4; ++i) {
        for (int j = 0; j < 4; ++j) {
          int32_t s = _mm512_reduce_add_epi32(c[i * 4 + j]);
          /* vector part used a+128: remove 128 * sum over the vector k range */
          int32_t tail = 0, wv = 0;
          for (int64_t k = K64; k < K; ++k)
            tail += (int32_t)ar[i][k] * (int32_t)wr[j][k];
          if (K64 == K) {
            wv = wsum[n + j];
          } else {
            for (int64_t k = 0; k < K64; ++k) wv += wr[j][k];
          }
          acc[(m + i) * N + n + j] = s - 128 * wv + tail;
        }
      }
    }
    if (n < N) {
      for (int i = 0; i < 4; ++i)
        for (int64_t nn = n; nn < N; ++nn) {
          const int8_t* a = A + (m + i) * K;
          const int8_t* w = Wnk + nn * K;
          int32_t s = 0;
          for (int64_t k = 0; k < K; ++k) s += (int32_t)a[k] * (int32_t)w[k];
          acc[(m + i) * N + nn] = s;
        }
    }
  }
  if (m < m1) gemm_nt_rows_plain(A, Wnk, acc, m, m1, N, K);
}
#endif

int q8o_gemm_s32_fast(const int8_t* A, const int8_t* Wnk, int32_t* acc,
                      int64_t M, int64_t N, int64_t K) {
  int use_vnni = 0;
#if defined(__x86_64__)
  __builtin_cpu_init();
  use_vnni = __builtin_cpu_supports("avx512vnni") &&
             __builtin_cpu_supports("avx512bw") && K < (1 << 15);
#endif
  int32_t* wsum = NULL;
  if (use_vnni) {
    wsum = (int32_t*)malloc(sizeof(int32_t) * (size_t)(N > 0 ? N : 1));
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
      int32_t s = 0;
      for (int64_t k = 0; k < K; ++k) s += Wnk[n * K + k];
      wsum[n] = s;
    }
  }
  int nthreads = 1;
#ifdef _OPENMP
  nthreads = omp_get_max_threads();
#endif
  /* blocks of 4 rows keep the register-blocked kernel busy */
  const int64_t MB = 4;
  const int64_t nblk = (M + MB - 1) / MB;
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t b = 0; b < nblk; ++b) {
    int64_t m0 = b * MB, m1 = m0 + MB < M ? m0 + MB : M;
#if defined(__x86_64__)
    if (use_vnni) {
      gemm_nt_rows_vnni(A, Wnk, wsum, acc, m0, m1, N, K);
      continue;
    }
#endif
    gemm_nt_rows_plain(A, Wnk, acc, m0, m1, N, K);
  }
  free(wsum);
  return nthreads;
}

/* ------------------------------------------------------------------------ */
/* float helpers                                                             */
/* ------------------------------------------------------------------------ */
static inline float rne_f32(float v) {
  /* nearbyintf under FE_TONEAREST = round half to even; callers never change
   * the rounding mode, but be explicit like the reference's folder is
   * (disc/IR/hlo_disc_ops.cc:243-249). */
  int cur = fegetround();
  if (cur != FE_TONEAREST) fesetround(FE_TONEAREST);
  float r = nearbyintf(v);
  if (cur != FE_TONEAREST) fesetround(cur);
  return r;
}

static inline int8_t sat_round_s8(float d) {
  /* oneDNN saturate-then-round: clamp in float, then nearbyint */
  if (!(d >= -128.0f)) d = -128.0f; /* also catches NaN -> lower bound */
  if (d > 127.0f) d = 127.0f;
  return (int8_t)rne_f32(d);
}

static inline int32_t sat_round_s32(float d) {
  /* INT32_MAX is not a float; the largest float below 2^31 is 2147483520 */
  if (!(d >= -2147483648.0f)) d = -2147483648.0f;
  if (d > 2147483520.0f) d = 2147483520.0f;
  return (int32_t)rne_f32(d);
}

/* R: matmul.hpp:532-533 bias_scales[i] = (dst_coeff*bias_scale)/(s_x*s_w[i]) with
 * dst_coeff = bias_scale = 1.0f; the reorder (matmul.hpp:622-625) multiplies by
 * it, rounds to nearest even and saturates to s32. */
void q8o_bias_f32_to_s32(const float* bias, float sx, const float* sw,
                         int64_t n_sw, int32_t* b32, int64_t N) {
  for (int64_t n = 0; n < N; ++n) {
    float w = sw[n_sw > 1 ? n : 0];
    float denom = sx * w;
    float bs = (1.0f * 1.0f) / denom;
    float v = bias[n] * bs;
    b32[n] = sat_round_s32(v);
  }
}

/* R: matmul.hpp:534-535 op_scales[i] = (s_x*s_w[i])/(dst_coeff*s_o); oneDNN 2.x
 * post-processing order: (f32(acc) + f32(bias)) * scale, + dst zero point,
 * saturate, round. */
void q8o_requant_cpu(const int32_t* acc, int64_t M, int64_t N,
                     const int32_t* b32, float sx, const float* sw,
                     int64_t n_sw, float so, int32_t zo, int8_t* out) {
  float* os = (float*)malloc(sizeof(float) * (size_t)(N > 0 ? N : 1));
  for (int64_t n = 0; n < N; ++n) {
    float num = sx * sw[n_sw > 1 ? n : 0];
    float den = 1.0f * so;
    os[n] = num / den;
  }
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float d = (float)acc[m * N + n];
      if (b32) d = d + (float)b32[n];
      d = d * os[n];
      if (zo != 0) d = d + (float)zo;
      out[m * N + n] = sat_round_s8(d);
    }
  }
  free(os);
}

/* ------------------------------------------------------------------------ */
/* Fixed-point requantisation of the AArch64 path.                           */
/* R: ral/context/common_context_impl_quantization.cc:671-679 (per channel), */
/*    :865-872 and :1083-1090 (per tensor) select                            */
/*    GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT and call             */
/*    arm_compute::quantization::calculate_quantized_multipliers.  The       */
/*    arithmetic itself lives in Arm Compute Library v23.02.1 (an            */
/*    http_archive of R/tao/third_party/..., blade_disc_dnn_workspace.bzl    */
/*    :27-38; its sources are not in the reference tree).  What follows      */
/*    restates the library's published algorithm:                            */
/*      multiplier[n] = s_x * s_w[n] / s_o              (binary32)           */
/*      frexp(multiplier) = q * 2^e, q in [0.5, 1);  M0 = round(q * 2^31),   */
/*      shift = -e  (M0 == 2^31 -> M0 /= 2, shift -= 1)                      */
/*      (AsymmHelpers.cpp: calculate_quantized_multiplier[_less_than_one |   */
/*       _greater_than_one])                                                 */
/*      v = acc + bias;                                                      */
/*      shift >= 0: v = rounding_divide_by_pow2(sqrdmulh(v, M0), shift)      */
/*      shift <  0: v = sqrdmulh(v * 2^-shift, M0)         (NEAsymm.h:       */
/*      finalize_quantization), v += z_o, clamp to [-128, 127].              */
/*    sqrdmulh is the AArch64 instruction the library's vqrdmulhq_n_s32      */
/*    compiles to: (2 a b + 2^31) >> 32, saturated; rounding_divide_by_pow2  */
/*    rounds half away from zero.  Parity beyond this published algorithm    */
/*    is unpinned: the reference holds no vectors for it but the 12.0 /      */
/*    108.0 closed forms of its AArch64 tests.                               */
/* ------------------------------------------------------------------------ */
int32_t q8o_sqrdmulh(int32_t a, int32_t b) {
  if (a == INT32_MIN && b == INT32_MIN) return INT32_MAX;
  const int64_t prod = (int64_t)a * (int64_t)b;
  /* (2 prod + 2^31) >> 32 with an arithmetic shift, written without overflow */
  const int64_t t = prod + ((int64_t)1 << 30);
  return (int32_t)(t >> 31);
}

int32_t q8o_rounding_divide_by_pow2(int32_t x, int exponent) {
  if (exponent <= 0) return x;
  if (exponent > 31) exponent = 31;
  const int32_t mask = (int32_t)(((uint32_t)1 << exponent) - 1u);
  const int32_t threshold = (mask >> 1) + (x < 0 ? 1 : 0);
  return (x >> exponent) + ((x & mask) > threshold ? 1 : 0);
}

void q8o_fixedpoint_multiplier(float multiplier, int32_t* quant_multiplier, int32_t* shift) {
  int e = 0;
  const double q = frexp((double)multiplier, &e);
  int64_t q_fixed = (int64_t)round(q * (double)((int64_t)1 << 31));
  int sh = -e;
  if (q_fixed == ((int64_t)1 << 31)) {
    q_fixed /= 2;
    --sh;
  }
  *quant_multiplier = (int32_t)q_fixed;
  *shift = sh;
}

int8_t q8o_finalize_fixedpoint(int32_t v, int32_t quant_multiplier, int32_t shift, int32_t zo) {
  if (shift < 0) {
    /* vmulq_n_s32: the product wraps */
    const int32_t scaled = (int32_t)((uint32_t)v * ((uint32_t)1 << (-shift > 31 ? 31 : -shift)));
    v = q8o_sqrdmulh(scaled, quant_multiplier);
  } else {
    v = q8o_rounding_divide_by_pow2(q8o_sqrdmulh(v, quant_multiplier), shift);
  }
  v = (int32_t)((uint32_t)v + (uint32_t)zo);
  if (v < -128) v = -128;
  if (v > 127) v = 127;
  return (int8_t)v;
}

void q8o_requant_fixedpoint(const int32_t* acc, int64_t M, int64_t N, const int32_t* b32,
                            float sx, const float* sw, int64_t n_sw, float so, int32_t zo,
                            int8_t* out) {
  int32_t* mult = (int32_t*)malloc(sizeof(int32_t) * (size_t)(N > 0 ? N : 1));
  int32_t* shift = (int32_t*)malloc(sizeof(int32_t) * (size_t)(N > 0 ? N : 1));
  for (int64_t n = 0; n < N; ++n) {
    const float num = sx * sw[n_sw > 1 ? n : 0];
    const float multiplier = num / so;
    q8o_fixedpoint_multiplier(multiplier, &mult[n], &shift[n]);
  }
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      int32_t v = acc[m * N + n];
      if (b32) v = (int32_t)((uint32_t)v + (uint32_t)b32[n]);
      out[m * N + n] = q8o_finalize_fixedpoint(v, mult[n], shift[n], zo);
    }
  }
  free(mult);
  free(shift);
}

/* R: quantized_gpu_kernel_impl.cc:262-265 (per channel) / :385 (per tensor):
 * kernel_scale = input_scale * weight_scale / result_scale, then
 * D = kernel_scale * acc + bias, converted to int8 with round-to-nearest-even
 * and saturation (cublasLt CUDA_R_8I output with an f32 scale type). */
void q8o_requant_gpu(const int32_t* acc, int64_t M, int64_t N,
                     const float* bias_f32, const int8_t* bias_i8,
                     const float* sx, int64_t n_sx, const float* sw,
                     int64_t n_sw, const float* so, int64_t n_so, int8_t* out) {
  float* alpha = (float*)malloc(sizeof(float) * (size_t)(N > 0 ? N : 1));
  for (int64_t n = 0; n < N; ++n) {
    float t = sx[n_sx > 1 ? n : 0] * sw[n_sw > 1 ? n : 0];
    alpha[n] = t / so[n_so > 1 ? n : 0];
  }
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float d = alpha[n] * (float)acc[m * N + n];
      if (bias_f32) d = d + bias_f32[n];
      if (bias_i8) d = d + (float)bias_i8[n];
      out[m * N + n] = sat_round_s8(d);
    }
  }
  free(alpha);
}

void q8o_dequant_acc(const int32_t* acc, int64_t M, int64_t N, float sx,
                     const float* sw, int64_t n_sw, const float* bias,
                     float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float s = sx * sw[n_sw > 1 ? n : 0];
      float d = (float)acc[m * N + n] * s;
      if (bias) d = d + bias[n];
      out[m * N + n] = d;
    }
  }
}

/* ------------------------------------------------------------------------ */
/* quantize / dequantize                                                     */
/* ------------------------------------------------------------------------ */
static void store_q(void* out, int64_t i, int kind, double v) {
  /* v is already rounded and clamped to [qmin,qmax] */
  switch (kind) {
    case Q8O_I8: ((int8_t*)out)[i] = (int8_t)v; break;
    case Q8O_U8: ((uint8_t*)out)[i] = (uint8_t)v; break;
    case Q8O_I16: ((int16_t*)out)[i] = (int16_t)v; break;
    case Q8O_U16: ((uint16_t*)out)[i] = (uint16_t)v; break;
    /* the f32 images of the 32-bit limits lie one past the integer range (2^31, 2^32): the
     * conversion of such a clamped value saturates -- this build's definition, the
     * reference's mhlo.convert leaves it undefined */
    case Q8O_I32: ((int32_t*)out)[i] = v >= 2147483648.0 ? INT32_MAX : (int32_t)v; break;
    default: ((uint32_t*)out)[i] = v >= 4294967296.0 ? UINT32_MAX : (uint32_t)v; break;
  }
}

/* R: disc_lower_quantize_and_dequantize.cc:77-94 -- all in f32:
 * t0 = x / scale; t1 = t0 + f32(zp); t2 = round(t1); t3 = clamp(t2, f32(qmin),
 * f32(qmax)); out = convert(t3). */
void q8o_quantize_f32(const float* x, int64_t outer, int64_t nch, int64_t inner,
                      const float* scale, const int32_t* zp, int64_t n_q,
                      int64_t qmin, int64_t qmax, int round_mode, int out_kind,
                      void* out) {
  const float fmin = (float)qmin, fmax = (float)qmax;
  const int64_t total = outer * nch * inner;
  /* elements are independent: split the flat index range over the threads */
#pragma omp parallel for schedule(static) if (total > 65536)
  for (int64_t idx = 0; idx < total; ++idx) {
    const int64_t qi = n_q > 1 ? (idx / inner) % nch : 0;
    const float s = scale[qi];
    const float z = (float)zp[qi];
    float t0 = x[idx] / s;
    float t1 = t0 + z;
    float t2 = round_mode == Q8O_ROUND_HALF_TO_EVEN ? rne_f32(t1) : roundf(t1);
    /* mhlo.clamp(min, x, max) = min(max(x, lo), hi) */
    float t3 = t2 < fmin ? fmin : t2;
    t3 = t3 > fmax ? fmax : t3;
    store_q(out, idx, out_kind, (double)t3);
  }
}

/* R: hlo_disc_ops.cc:286-309 -- double: x/scale + zp, nearbyint narrowed through
 * float (":246 float roundVal = std::nearbyint(val)") or std::round, clamp. */
void q8o_quantize_fold(const float* x, int64_t outer, int64_t nch,
                       int64_t inner, const float* scale, const int32_t* zp,
                       int64_t n_q, int64_t qmin, int64_t qmax, int round_mode,
                       int out_kind, void* out) {
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t c = 0; c < nch; ++c) {
      int64_t qi = n_q > 1 ? c : 0;
      double s = (double)scale[qi];
      int64_t z = zp[qi];
      for (int64_t i = 0; i < inner; ++i) {
        int64_t idx = (o * nch + c) * inner + i;
        double d = ((double)x[idx] / s) + (double)z;
        double r;
        if (round_mode == Q8O_ROUND_HALF_TO_EVEN) {
          float rv = (float)nearbyint(d);
          r = (double)rv;
        } else {
          r = round(d);
        }
        if (r < (double)qmin) r = (double)qmin;
        if (r > (double)qmax) r = (double)qmax;
        store_q(out, idx, out_kind, r);
      }
    }
}

/* R: disc_lower_quantize_and_dequantize.cc:131-136 -- convert q to the zero point's
 * integer type, subtract, convert to f32, multiply by scale. */
void q8o_dequantize(const void* q, int in_kind, int64_t outer, int64_t nch,
                    int64_t inner, const float* scale, const int32_t* zp,
                    int64_t n_q, float* out) {
  const int64_t total = outer * nch * inner;
#pragma omp parallel for schedule(static) if (total > 65536)
  for (int64_t idx = 0; idx < total; ++idx) {
    const int64_t qi = n_q > 1 ? (idx / inner) % nch : 0;
    int32_t v;
    switch (in_kind) {
      case Q8O_I8: v = ((const int8_t*)q)[idx]; break;
      case Q8O_U8: v = ((const uint8_t*)q)[idx]; break;
      case Q8O_I16: v = ((const int16_t*)q)[idx]; break;
      case Q8O_U16: v = ((const uint16_t*)q)[idx]; break;
      default: v = ((const int32_t*)q)[idx]; break;
    }
    int32_t t0 = v - zp[qi];
    out[idx] = (float)t0 * scale[qi];
  }
}

/* ------------------------------------------------------------------------ */
/* convolution                                                               */
/* R: metadata layout disc_lower_to_library_call.cc:273-336; operand meaning  */
/*    stream_executor_based_impl.cc:1831-1841                                */
/* ------------------------------------------------------------------------ */
static void strides_of(const int64_t sizes[4], int64_t st[4]) {
  st[3] = 1;
  for (int i = 3; i > 0; --i) st[i - 1] = st[i] * sizes[i];
}

void q8o_conv_s32(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                  const int64_t w_sizes[4], const int32_t padding[4],
                  const int32_t md[17], int32_t* acc,
                  const int64_t out_sizes[4], int32_t zx, int32_t zw) {
  int64_t ist[4], wst[4], ost[4];
  strides_of(in_sizes, ist);
  strides_of(w_sizes, wst);
  strides_of(out_sizes, ost);
  const int ib = md[0], ic = md[1], ih = md[2], iw = md[3];
  const int ki = md[4], ko = md[5], kh = md[6], kw = md[7];
  const int ob = md[8], oc = md[9], oh = md[10], ow = md[11];
  const int64_t sh = md[12], sw_ = md[13], dh = md[14], dw = md[15];
  const int64_t NB = in_sizes[ib], CI = in_sizes[ic], H = in_sizes[ih],
                W = in_sizes[iw];
  const int64_t CO = w_sizes[ko], KH = w_sizes[kh], KW = w_sizes[kw];
  const int64_t HO = out_sizes[oh], WO = out_sizes[ow];
  const int64_t total = NB * HO * WO;
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < total; ++p) {
    int64_t b = p / (HO * WO), y = (p / WO) % HO, x = p % WO;
    for (int64_t co = 0; co < CO; ++co) {
      int32_t s = 0;
      for (int64_t r = 0; r < KH; ++r) {
        int64_t yy = y * sh - padding[0] + r * dh;
        for (int64_t q = 0; q < KW; ++q) {
          int64_t xx = x * sw_ - padding[2] + q * dw;
          int inside = yy >= 0 && yy < H && xx >= 0 && xx < W;
          for (int64_t ci = 0; ci < CI; ++ci) {
            /* padded positions hold the input zero point, i.e. contribute
             * (zx - zx) = 0 */
            if (!inside) continue;
            int32_t a =
                in[b * ist[ib] + ci * ist[ic] + yy * ist[ih] + xx * ist[iw]];
            int32_t v =
                w[ci * wst[ki] + co * wst[ko] + r * wst[kh] + q * wst[kw]];
            s += (a - zx) * (v - zw);
          }
        }
      }
      acc[b * ost[ob] + co * ost[oc] + y * ost[oh] + x * ost[ow]] = s;
    }
  }
}

/* R: common_context_impl_quantization.h:47-62 */
int q8o_conv_reorder_dims(const char* fmt, int32_t reorder[4]) {
  const char* pn = strchr(fmt, 'N');
  const char* pc = strchr(fmt, 'C');
  if (!pn || !pc) return 0;
  int32_t b = (int32_t)(pn - fmt), c = (int32_t)(pc - fmt);
  int idx = 0;
  for (int i = 0; i < 4; ++i) {
    if (i == b || i == c) continue;
    if (idx < 4) reorder[idx] = i;
    idx++;
  }
  if (idx != 2) return 0;
  reorder[2] = b;
  reorder[3] = c;
  return 1;
}

/* R: :64-98 (generateStrides / generateDilations share one rule) */
int q8o_conv_expand(const int32_t reorder[4], const int64_t* arr, int64_t n,
                    int32_t out2[2]) {
  if (n == 1) {
    out2[0] = out2[1] = (int32_t)arr[0];
  } else if (n == 2) {
    out2[0] = (int32_t)arr[0];
    out2[1] = (int32_t)arr[1];
  } else if (n == 4) {
    out2[0] = (int32_t)arr[reorder[0]];
    out2[1] = (int32_t)arr[reorder[1]];
  } else {
    return 0;
  }
  return 1;
}

/* R: :100-135 (TF SAME / VALID) */
int q8o_conv_padding(const int64_t in_sizes[4], const int64_t w_sizes[4],
                     const char* padding, const int32_t reorder[4],
                     const int32_t strides[2], const int32_t dilations[2],
                     int32_t pad[4]) {
  if (strcmp(padding, "SAME") == 0) {
    for (int i = 0; i < 2; ++i) {
      int in_sz = (int)in_sizes[reorder[i]];
      int k = (int)w_sizes[i + 1];
      int keff = (k - 1) * dilations[i] + 1;
      int along;
      if (in_sz % strides[i] == 0)
        along = keff - strides[i];
      else
        along = keff - (in_sz % strides[i]);
      if (along < 0) along = 0;
      pad[2 * i] = along / 2;
      pad[2 * i + 1] = along - pad[2 * i];
    }
    return 1;
  }
  if (strcmp(padding, "VALID") == 0) {
    pad[0] = pad[1] = pad[2] = pad[3] = 0;
    return 1;
  }
  return 0;
}

/* R: :137-157 */
int q8o_conv_explicit_padding(const int32_t reorder[4], const int64_t* ep,
                              int64_t n, int32_t pad[4]) {
  if (n == 4) {
    for (int i = 0; i < 4; ++i) pad[i] = (int32_t)ep[i];
    return 1;
  }
  if (n == 8) {
    for (int i = 0; i < 2; ++i) {
      pad[2 * i] = (int32_t)ep[2 * reorder[i]];
      pad[2 * i + 1] = (int32_t)ep[2 * reorder[i] + 1];
    }
    return 1;
  }
  return 0;
}

/* R: :159-186 */
int q8o_conv_metadata(const int32_t strides[2], const int32_t dilations[2],
                      const int32_t reorder[4], int weight_is_const,
                      int32_t md[17]) {
  int i = 0;
  md[i++] = reorder[2];
  md[i++] = reorder[3];
  md[i++] = reorder[0];
  md[i++] = reorder[1];
  md[i++] = 3; /* kernel input features: last dim (OHWI) */
  md[i++] = 0; /* kernel output features */
  md[i++] = 1;
  md[i++] = 2;
  md[i++] = reorder[2];
  md[i++] = reorder[3];
  md[i++] = reorder[0];
  md[i++] = reorder[1];
  md[i++] = strides[0];
  md[i++] = strides[1];
  md[i++] = dilations[0];
  md[i++] = dilations[1];
  md[i++] = weight_is_const ? 1 : 0;
  return i == 17;
}

/* R: :188-206 */
void q8o_conv_result_shape(const int64_t in_sizes[4], const int64_t w_sizes[4],
                           const int32_t reorder[4], const int32_t pad[4],
                           const int32_t strides[2], const int32_t dilations[2],
                           int64_t out_sizes[4]) {
  for (int i = 0; i < 2; ++i) {
    int rank = reorder[i];
    int ori = (int)in_sizes[rank];
    int k = (int)w_sizes[i + 1];
    int s = strides[i], d = dilations[i];
    int p1 = pad[2 * i], p2 = pad[2 * i + 1];
    out_sizes[rank] = (ori + p1 + p2 - k * d + d + s - 1) / s;
  }
  out_sizes[reorder[2]] = in_sizes[reorder[2]];
  out_sizes[reorder[3]] = w_sizes[0];
}
