/*
 * q8_oracle.h -- CPU restatement of BladeDISC's quantized-inference hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared against and the timed CPU baseline of the benchmark.  Nothing in the
 * shipped GPU path links, loads or calls it.
 *
 * Every function restates an algorithm of the reference (R = alibaba/BladeDISC,
 * paths relative to tao_compiler/mlir/):
 *
 *   q8o_gemm_s32            int32 accumulation of an s8 x s8 matmul, as requested
 *                           from oneDNN by ral/context/common_context_impl_quantization.cc
 *                           :1196-1266 (layouts from tp_a/tp_b at :1219-1234).
 *   q8o_bias_f32_to_s32     the f32 -> s32 bias reorder with bias_scales[n] =
 *                           1/(s_x*s_w[n]): ral/context/mkldnn/ideep/ideep/operators/
 *                           matmul.hpp:532-533,556-565 (attr) and :622-625 (reorder).
 *   q8o_requant_cpu  (E1)   out = sat8(rne((f32(acc)+f32(b32[n])) * os[n] + z_o)),
 *                           os[n] = (s_x*s_w[n])/(1*s_o): matmul.hpp:534-535; the
 *                           order "add bias, multiply by the output scale, add the
 *                           destination zero point, saturate, round-to-nearest-even"
 *                           is oneDNN 2.x's documented int8 matmul post-processing
 *                           (oneDNN is an un-vendored submodule of the reference,
 *                           version 2.x by API: dnnl::primitive_attr::set_output_scales).
 *   q8o_requant_gpu  (E2)   out = sat8(rne(alpha[n]*f32(acc) + bias[n])), alpha =
 *                           s_x*s_w/s_o evaluated left to right:
 *                           ral/context/quantized_gpu_kernel_impl.cc:262-265,385,416-420
 *                           (cublasLt alpha + EPILOGUE_BIAS) and
 *                           ral/context/stream_executor_based_impl.cc:458.
 *   q8o_requant_fixedpoint  the AArch64 path's requantisation by a fixed-point multiplier
 *                           and shift (GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT,
 *                           ral/context/common_context_impl_quantization.cc:671-679,
 *                           865-872, 1083-1090); the arithmetic is Arm Compute Library's
 *                           (v23.02.1, not in the reference tree): published algorithm
 *                           restated, PARITY UNPINNED beyond it.
 *   q8o_dequant_acc  (E3)   f32(acc)*(s_x*s_w[n]) + bias[n]: qgemm followed by
 *                           mhlo_disc.dequantize with a per-channel scale.
 *   q8o_quantize_f32        disc/transforms/disc_lower_quantize_and_dequantize.cc:77-94
 *                           (f32 divide, add zp, round, clamp, convert).
 *   q8o_quantize_fold       disc/IR/hlo_disc_ops.cc:227-340 (the compile-time folder:
 *                           same formula in double).
 *   q8o_dequantize          disc/transforms/disc_lower_quantize_and_dequantize.cc:131-136.
 *   q8o_conv_s32            int32 accumulation of the convolution described by the
 *                           ral_qconv metadata vector (disc/transforms/
 *                           disc_lower_to_library_call.cc:273-336).
 *   q8o_conv_* helpers      ral/context/common_context_impl_quantization.h:47-206.
 *
 * Parity status: integer accumulation, quantize, dequantize and the conv helpers are
 * pinned by the reference's own known-answer tests and golden vectors.  The last-bit
 * behaviour of E1 lives in oneDNN 2.x, which is absent from the reference checkout:
 * E1 is "parity unpinned" beyond the reference's closed-form cases (12.0 / 108.0 /
 * 128.0) and the scale algebra visible at the ideep call sites.
 */
#ifndef Q8_ORACLE_H_
#define Q8_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* round modes of mhlo_disc.quantize (disc/IR/hlo_disc_enums.td) */
#define Q8O_ROUND_HALF_AWAY_FROM_ZERO 0
#define Q8O_ROUND_HALF_TO_EVEN 1

/* output element kinds of quantize / input kinds of dequantize */
#define Q8O_I8 0
#define Q8O_U8 1
#define Q8O_I16 2
#define Q8O_U16 3
#define Q8O_I32 4
#define Q8O_U32 5

/* acc[m,n] = sum_k (A(m,k)-zx) * (W(k,n)-zw).
 * A is [M,K] row-major (tp_a=0) or [K,M] row-major (tp_a=1);
 * W is [K,N] row-major (tp_b=0) or [N,K] row-major (tp_b=1). */
void q8o_gemm_s32(const int8_t* A, const int8_t* W, int32_t* acc, int64_t M,
                  int64_t N, int64_t K, int tp_a, int tp_b, int32_t zx,
                  int32_t zw);

/* Same result as q8o_gemm_s32(tp_a=0,tp_b=1,zx=zw=0); OpenMP + AVX512-VNNI when
 * the host has it.  Used for large parity cases and as the timed CPU baseline.
 * Returns the number of threads used. */
int q8o_gemm_s32_fast(const int8_t* A, const int8_t* Wnk, int32_t* acc,
                      int64_t M, int64_t N, int64_t K);

/* b32[n] = sat_s32(rne(bias[n] * (1.0f / (sx * sw[n or 0])))) */
void q8o_bias_f32_to_s32(const float* bias, float sx, const float* sw,
                         int64_t n_sw, int32_t* b32, int64_t N);

/* E1.  b32 may be NULL (no bias).  n_sw is 1 (per tensor) or N. */
void q8o_requant_cpu(const int32_t* acc, int64_t M, int64_t N,
                     const int32_t* b32, float sx, const float* sw,
                     int64_t n_sw, float so, int32_t zo, int8_t* out);

/* E2.  Exactly one of bias_f32 / bias_i8 may be non-NULL (or none).
 * Each of n_sx / n_sw / n_so is 1 (rank-0 scale) or N (per-channel vector). */
void q8o_requant_gpu(const int32_t* acc, int64_t M, int64_t N,
                     const float* bias_f32, const int8_t* bias_i8,
                     const float* sx, int64_t n_sx, const float* sw,
                     int64_t n_sw, const float* so, int64_t n_so, int8_t* out);

/* Fixed-point requantisation (see q8_oracle.c for the algorithm and its source).
 *   q8o_sqrdmulh               saturating rounding doubling multiply, high half
 *   q8o_rounding_divide_by_pow2  x / 2^exponent, ties away from zero
 *   q8o_fixedpoint_multiplier  multiplier -> (M0 in [2^30, 2^31), shift), multiplier =
 *                              M0 * 2^-31 * 2^-shift exactly (a binary32 has 24 bits)
 *   q8o_finalize_fixedpoint    one value through the output stage
 *   q8o_requant_fixedpoint     out = clamp8(stage(acc + b32[n], M0[n], shift[n]) + zo),
 *                              multiplier[n] = (sx * sw[n]) / so in binary32; b32 may be NULL */
int32_t q8o_sqrdmulh(int32_t a, int32_t b);
int32_t q8o_rounding_divide_by_pow2(int32_t x, int exponent);
void q8o_fixedpoint_multiplier(float multiplier, int32_t* quant_multiplier, int32_t* shift);
int8_t q8o_finalize_fixedpoint(int32_t v, int32_t quant_multiplier, int32_t shift, int32_t zo);
void q8o_requant_fixedpoint(const int32_t* acc, int64_t M, int64_t N, const int32_t* b32,
                            float sx, const float* sw, int64_t n_sw, float so, int32_t zo,
                            int8_t* out);

/* E3.  bias may be NULL. */
void q8o_dequant_acc(const int32_t* acc, int64_t M, int64_t N, float sx,
                     const float* sw, int64_t n_sw, const float* bias,
                     float* out);

/* x viewed as [outer, nch, inner]; scale/zp have n_q = 1 or nch entries. */
void q8o_quantize_f32(const float* x, int64_t outer, int64_t nch, int64_t inner,
                      const float* scale, const int32_t* zp, int64_t n_q,
                      int64_t qmin, int64_t qmax, int round_mode, int out_kind,
                      void* out);
void q8o_quantize_fold(const float* x, int64_t outer, int64_t nch,
                       int64_t inner, const float* scale, const int32_t* zp,
                       int64_t n_q, int64_t qmin, int64_t qmax, int round_mode,
                       int out_kind, void* out);
void q8o_dequantize(const void* q, int in_kind, int64_t outer, int64_t nch,
                    int64_t inner, const float* scale, const int32_t* zp,
                    int64_t n_q, float* out);

/* Convolution int32 accumulators for rank-4 tensors.
 * metadata (17 x i32): input {batch,channel,sp0,sp1}, kernel {in,out,sp0,sp1},
 * output {batch,channel,sp0,sp1}, strides[2], dilations[2], weight_is_const.
 * padding (4 x i32): {lo0,hi0,lo1,hi1}.  acc has the output layout. */
void q8o_conv_s32(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                  const int64_t w_sizes[4], const int32_t padding[4],
                  const int32_t metadata[17], int32_t* acc,
                  const int64_t out_sizes[4], int32_t zx, int32_t zw);

/* TF-style attribute helpers; all return 1 on success, 0 on failure. */
int q8o_conv_reorder_dims(const char* data_format, int32_t reorder[4]);
int q8o_conv_expand(const int32_t reorder[4], const int64_t* arr, int64_t n,
                    int32_t out2[2]); /* strides or dilations */
int q8o_conv_padding(const int64_t in_sizes[4], const int64_t w_sizes[4],
                     const char* padding, const int32_t reorder[4],
                     const int32_t strides[2], const int32_t dilations[2],
                     int32_t pad[4]);
int q8o_conv_explicit_padding(const int32_t reorder[4], const int64_t* ep,
                              int64_t n, int32_t pad[4]);
int q8o_conv_metadata(const int32_t strides[2], const int32_t dilations[2],
                      const int32_t reorder[4], int weight_is_const,
                      int32_t metadata[17]);
void q8o_conv_result_shape(const int64_t in_sizes[4], const int64_t w_sizes[4],
                           const int32_t reorder[4], const int32_t pad[4],
                           const int32_t strides[2], const int32_t dilations[2],
                           int64_t out_sizes[4]);

#ifdef __cplusplus
}
#endif
#endif /* Q8_ORACLE_H_ */
