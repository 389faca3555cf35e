/*
 * disc_q8.h -- C ABI of the MI355X (gfx950) quantized-inference kernels.
 *
 * These are the launchers the RAL entries in include/tao_ral_api.h are built on.
 * Every pointer marked "device" is HBM-resident; nothing here dereferences a
 * device pointer on the host, synchronises a stream, or allocates memory.
 * All launches go to `stream` (a hipStream_t passed as void*; NULL = the null
 * stream).  Return value: 0 on success, non-zero on error with the message
 * available from dq8_last_error() (thread-local).
 *
 * Reference interfaces replaced (R = alibaba/BladeDISC, tao_compiler/mlir/):
 *   dq8_qgemm      -> the vendor GEMM behind ral_qgemm
 *                     (R ral/context/stream_executor_based_impl.cc:427-483, bladnn::gemm)
 *                     and behind ral_pdll_qgemm[_per_channel]
 *                     (R ral/context/quantized_gpu_kernel_impl.cc:129-158 cublasLtMatmul,
 *                     :197-321, :329-422), plus the CPU-signature variants
 *                     (R ral/context/common_context_impl_quantization.cc:1196-1672).
 *   dq8_qconv2d    -> the fused int8 convolution behind ral_qconv
 *                     (R ral/context/stream_executor_based_impl.cc:1506-1588, 1831-1948).
 *   dq8_minmax     -> torch.aminmax in the calibration observers
 *                     (R tools/torch_quant/torch_quant/observer.py:236-241, 261-281).
 *   dq8_quantize / dq8_dequantize
 *                  -> the loops the compiler generates from mhlo_disc.quantize /
 *                     mhlo_disc.dequantize
 *                     (R disc/transforms/disc_lower_quantize_and_dequantize.cc:36-139, 141-215).
 *   dq8_tf_quantize_v2 / dq8_tf_dequantize
 *                  -> the loops the compiler generates from tf.QuantizeV2 / tf.Dequantize
 *                     (R disc/transforms/lower_tf.cc:307-560, 562-654).
 */
#ifndef DISC_Q8_H_
#define DISC_Q8_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- enums (plain ints in the ABI) ------------------------------------ */

/* epilogue applied to the int32 accumulators */
#define DQ8_EPI_ACC_S32 0     /* out: int32  acc                                          */
#define DQ8_EPI_REQUANT_CPU 1 /* out: int8   sat(rne((f32(acc)+b32[n])*os[n] + zo))        */
#define DQ8_EPI_REQUANT_GPU 2 /* out: int8   sat(rne(os[n]*f32(acc) + bias[n]))            */
#define DQ8_EPI_DEQUANT_F32 3 /* out: float  f32(acc)*(sx*sw[n]) + bias[n]                 */
/* dq8_qgemm and dq8_qconv2d: the int8 result q of REQUANT_CPU / REQUANT_GPU dequantized in the same
 * epilogue, out: float (float)(q - zo) * so -- bit for bit what dq8_dequantize makes of the
 * requantized output, without the int8 round trip through memory.  Per-tensor `so` only;
 * bias kinds and zero points as for the requant form. */
#define DQ8_EPI_REQUANT_CPU_DEQUANT_F32 4
#define DQ8_EPI_REQUANT_GPU_DEQUANT_F32 5
/* os[n] = (sx*sw[n])/so evaluated in binary32, left to right.                            */
/* dq8_qgemm and dq8_qconv2d: the integer output stage of the reference's AArch64 path
 * (R ral/context/common_context_impl_quantization.cc:671-679, 865-872, 1083-1090:
 * GEMMLowpOutputStageType::QUANTIZE_DOWN_FIXEDPOINT of Arm Compute Library), out: int8
 *   multiplier[n] = (sx*sw[n])/so in binary32 = M0[n] 2^-31 2^-shift[n], M0 in [2^30, 2^31)
 *   v = acc + bias[n];  shift >= 0: v = rdivpot(sqrdmulh(v, M0), shift)
 *                       shift <  0: v = sqrdmulh(v 2^-shift, M0)
 *   out = clamp(v + zo, -128, 127)
 * with sqrdmulh(a, b) = (2ab + 2^31) >> 32 and rdivpot rounding ties away from zero.  Bias:
 * none or DQ8_BIAS_S32; sx and so per tensor, sw per tensor or per channel.  Not bit-identical
 * to the float stages (different rounding), by design of the reference's two CPU paths. */
#define DQ8_EPI_REQUANT_FIXEDPOINT 6

/* bias operand kinds */
#define DQ8_BIAS_NONE 0
#define DQ8_BIAS_S32 1 /* REQUANT_CPU: used as is                                          */
#define DQ8_BIAS_F32 2 /* REQUANT_CPU: b32 = sat32(rne(bias/(sx*sw[n]))) first;
                          REQUANT_GPU / DEQUANT_F32: added as is                           */
#define DQ8_BIAS_S8 3  /* REQUANT_GPU: (float)bias                                          */

/* element kinds of quantized tensors */
/* floating-point element types (dq8_quantize_ex, dq8_weight_only_qgemm) */
#define DQ8_DTYPE_F32 0
#define DQ8_DTYPE_F16 1
#define DQ8_I8 0
#define DQ8_U8 1
/* (dq8_quantize_ex / dq8_dequantize_ex only) */
#define DQ8_I16 2
#define DQ8_U16 3
#define DQ8_I32 4
#define DQ8_U32 5

/* mhlo_disc round_mode (R disc/IR/hlo_disc_enums.td) */
#define DQ8_ROUND_HALF_AWAY_FROM_ZERO 0
#define DQ8_ROUND_HALF_TO_EVEN 1

/* tf.QuantizeV2 modes */
#define DQ8_TF_SCALED 0
#define DQ8_TF_MIN_FIRST 1

/* ---- library ---------------------------------------------------------- */

const char* dq8_last_error(void);
/* packed version: major*10000 + minor*100 + patch */
int dq8_version(void);
/* Number of compute units / LDS bytes / clock the library sees on the current
 * device; fills what it can, returns 0 on success. */
int dq8_device_info(int* compute_units, int* lds_bytes_per_cu, int* clock_khz);

/* dst[0 .. bytes) = (uint8_t)value, as a kernel launch (any alignment).  What the runtime's
 * ral_gpu_memset issues in place of the reference's cudaMemsetAsync
 * (R ral/context/base/cuda/cuda_context_impl.cc:272-281): a compiled program whose execution
 * is captured into a HIP graph then records a kernel node, not a memset node. */
int dq8_fill(void* dst, int value, size_t bytes, void* stream);

/* ---- calibration statistics -------------------------------------------- */

/* Running minimum and maximum of a float tensor, per tensor or per channel: what the
 * reference's calibration observers accumulate before they derive scales and zero points
 * (R tools/torch_quant/torch_quant/observer.py:236-241 MinMaxObserver via torch.aminmax,
 * :261-281 PerChannelMinMaxObserver).  x (device, f32) is viewed as [outer, channels, inner];
 * for every channel c
 *     min_io[c] = min(min_io[c], min over o, i of x[o, c, i])
 *     max_io[c] = max(max_io[c], max ...)
 * so the caller keeps the observer's state in min_io / max_io (device f32, `channels`
 * entries, +inf / -inf before anything has been observed).  A NaN in a channel's data makes
 * both of its values NaN, as torch.aminmax does.  An empty tensor leaves the state as it is.
 * `workspace` (device) must hold dq8_minmax_workspace_bytes(...) bytes. */
size_t dq8_minmax_workspace_bytes(int64_t outer, int64_t channels, int64_t inner);
int dq8_minmax(const float* x, int64_t outer, int64_t channels, int64_t inner, float* min_io,
               float* max_io, void* workspace, size_t workspace_bytes, void* stream);

/* dq8_minmax without a workspace argument and without any allocation: no hipMalloc, hipFree
 * or allocating library routine is called.  No counterpart in the reference; it is for
 * callers that cannot allocate -- code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  The (min, max) pairs of the first pass go to an array
 * of dq8_minmax_static_max_bytes() bytes (4 MiB) that the library holds in the memory of
 * every device it runs on until the process ends; a tensor that needs more
 * (dq8_minmax_workspace_bytes() tells) is refused with an error and must use dq8_minmax.
 * Same results as dq8_minmax, bit for bit.  All calls on one device share that array:
 * calls that overlap on one device (different streams, different threads) race; calls on
 * one stream are ordered and safe.  Nothing in the array needs clearing between calls
 * (the first pass writes every pair the second reads). */
size_t dq8_minmax_static_max_bytes(void);
int dq8_minmax_static(const float* x, int64_t outer, int64_t channels, int64_t inner,
                      float* min_io, float* max_io, void* stream);

/* ---- quantize / dequantize -------------------------------------------- */

/* x (device, f32) is viewed as [outer, nch, inner]; scale (device f32) and zp
 * (device i32) hold n_q = 1 (per tensor) or nch (per channel along the middle
 * axis) entries.  out[i] = convert(clamp(round(x[i]/scale + (f32)zp), qmin, qmax)). */
int dq8_quantize(const float* x, void* out, int out_kind, int64_t outer,
                 int64_t nch, int64_t inner, const float* scale,
                 const int32_t* zp, int64_t n_q, int32_t qmin, int32_t qmax,
                 int round_mode, void* stream);

/* out[i] = (f32)((i32)q[i] - zp) * scale */
int dq8_dequantize(const void* q, int in_kind, float* out, int64_t outer,
                   int64_t nch, int64_t inner, const float* scale,
                   const int32_t* zp, int64_t n_q, void* stream);

/* dq8_quantize / dq8_dequantize for every quantized type the reference's operator takes
 * (i8, ui8, i16, ui16, i32, ui32: R disc/transforms/tests/disc-fold-quantize.mlir:48-247) and,
 * beyond the reference (whose lowering refuses anything but f32 input,
 * R disc/transforms/disc_lower_quantize_and_dequantize.cc:46-48), f16 input, which is widened
 * to f32 exactly before the same steps.  x_dtype: DQ8_DTYPE_*; kinds: DQ8_I8 .. DQ8_U32.  The
 * conversion of the clamped f32 value saturates (the f32 images of 2^31 - 1 and 2^32 - 1 lie
 * one past the integer range).  f32 -> 8-bit forwards to dq8_quantize. */
int dq8_quantize_ex(const void* x, int x_dtype, void* out, int out_kind, int64_t outer,
                    int64_t nch, int64_t inner, const float* scale, const int32_t* zp,
                    int64_t n_q, int64_t qmin, int64_t qmax, int round_mode, void* stream);
int dq8_dequantize_ex(const void* q, int in_kind, float* out, int64_t outer, int64_t nch,
                      int64_t inner, const float* scale, const int32_t* zp, int64_t n_q,
                      void* stream);

/* Fake quantization: dq8_dequantize(dq8_quantize(x)) in one pass, f32 -> f32, without
 * the integer tensor in between; bit for bit the result of the two calls (what the
 * reference's observers apply while calibrating, R tools/torch_quant/torch_quant/
 * observer.py:181-208; the compiler rewrites mhlo_disc.fake_quant into exactly this pair,
 * R disc/transforms/disc_convert_fake_quant_op.cc).  Arguments as for dq8_quantize; qmin / qmax within [-32768, 65535].  out may be x. */
int dq8_fake_quant(const float* x, float* out, int64_t outer, int64_t nch, int64_t inner,
                   const float* scale, const int32_t* zp, int64_t n_q, int32_t qmin,
                   int32_t qmax, int round_mode, void* stream);

/* ---- elementwise function between two quantized tensors ----------------- */

/* out[i] = table[in[i]] over n bytes (device; in == out allowed), `table` = 256 device bytes
 * indexed by the input byte's bit pattern (for int8 data: index (uint8_t)q).  The compiler
 * fuses dequantize -> activation -> quantize chains between two quantized operators into one
 * generated kernel (R disc/transforms/disc_lower_quantize_and_dequantize.cc lowers both ends
 * to elementwise ops that the fusion pass merges with the activation); since the chain's
 * input takes at most 256 values, its result is exactly a table, whatever the activation. */
int dq8_lut8(const void* in, void* out, int64_t n, const void* table, void* stream);

/* ---- TensorFlow's QuantizeV2 / Dequantize ------------------------------ */

/* tf.QuantizeV2 as the reference lowers it (R disc/transforms/lower_tf.cc:307-560): x
 * (device, f32) is viewed as [outer, channels, inner]; min_range / max_range (device f32)
 * hold `channels` entries (1 = per tensor, the op's axis = -1).  For every channel the range
 * is first adjusted (R :365-393: extended to contain zero and to be at least
 * ensure_minimum_range * max(|min|, |max|, 1) wide), then
 *   DQ8_TF_SCALED    (R :453-560)  f = min(min_q / min', max_q / max') over the sides whose
 *                    product with the bound is positive, min_q = lowest + narrow_range;
 *                    q = (T) round(clamp(x, min_q / f, max_q / f) * f);
 *                    out_min / out_max = min_q / f, max_q / f
 *   DQ8_TF_MIN_FIRST (R :395-451, channels = 1 only) r = (max' - min') / 255;
 *                    q = (T) clamp(round(x r) - (round(min' r) - lowest), lowest, highest);
 *                    out_min / out_max = min', max'
 * Every step is a separately rounded f32 operation; round is tf.Round (half to even), the
 * only rounding the reference's pattern accepts (it refuses round_mode HALF_TO_EVEN, whose
 * TF kernel differs, and mode MIN_COMBINED).  out_min / out_max (device f32, `channels`
 * entries) are the op's second and third results.  `params` (device, 16-byte aligned,
 * dq8_tf_params_bytes(channels) bytes) is working storage; after the call its float
 * [4 c + 2] is the factor channel c was multiplied by. */
size_t dq8_tf_params_bytes(int64_t channels);
int dq8_tf_quantize_v2(const float* x, void* out, int out_kind, int64_t outer, int64_t channels,
                       int64_t inner, const float* min_range, const float* max_range, int mode,
                       int narrow_range, float ensure_minimum_range, float* out_min,
                       float* out_max, void* params, size_t params_bytes, void* stream);

/* tf.Dequantize, mode SCALED (R disc/transforms/lower_tf.cc:562-654):
 *   out = f[c] * (float) q,   f = max(min / min_q, max / highest) for int8 input,
 *                             f = max / 255 for uint8 input.
 * Same view and range operands as above; `params` as above (after the call its first
 * `channels` floats are f). */
int dq8_tf_dequantize(const void* q, int in_kind, float* out, int64_t outer, int64_t channels,
                      int64_t inner, const float* min_range, const float* max_range,
                      int narrow_range, void* params, size_t params_bytes, void* stream);

/* ---- int8 GEMM -------------------------------------------------------- */

/* Bytes of device scratch dq8_qgemm needs for this problem with zx == zw == 0 (0 when it
 * needs none: tp_a == 0, tp_b == 1 and K % 16 == 0).  Operands in the other layout, or with
 * a K that is not a multiple of 16, are rewritten there as [rows, K rounded up to 16].  A
 * ragged K without the scratch still gives the right result, from the generic kernel; a
 * transposed operand without it is an error. */
size_t dq8_qgemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int tp_a,
                                 int tp_b);
/* The same for given input / weight zero points: with a non-zero one it adds two correction
 * vectors (4 (M + N) bytes), which lets dq8_qgemm keep such a problem on the MFMA kernels.
 * A caller that passes less (but at least dq8_qgemm_workspace_bytes()) still gets the
 * right result, from the generic kernel. */
size_t dq8_qgemm_workspace_bytes_zp(int64_t M, int64_t N, int64_t K, int tp_a, int tp_b,
                                    int32_t zx, int32_t zw);

/* out[M,N] = epilogue( sum_k A(m,k) * W(k,n) ).
 *   A: device int8, [M,K] with row stride lda (tp_a = 0) or [K,M] with row
 *      stride lda (tp_a = 1).
 *   W: device int8, [N,K] row stride ldw (tp_b = 1, the GPU callers' layout) or
 *      [K,N] row stride ldw (tp_b = 0, the CPU callers' layout).
 *   out: device, element type per `epilogue`, row stride ldo (elements).
 *   sx / sw / so: device f32 with n_sx / n_sw / n_so entries, each 1 or N.
 *   zx / zw: input and weight zero points, acc = sum (A - zx) * (W - zw) (what oneDNN
 *      computes for the reference's CPU entries, R ral/context/mkldnn/ideep/ideep/
 *      operators/matmul.hpp:516-549: one source zero point, the first weight zero point).
 *      With scratch of dq8_qgemm_workspace_bytes_zp() the MFMA kernels start their sums at
 *      - zx sum_k W[n,k] - zw sum_k A[m,k] + K zx zw (row sums from a small kernel); with
 *      less scratch, or operands the MFMA kernels cannot take, the generic scalar kernel
 *      is used.
 *   zo: output zero point (REQUANT_CPU only).
 *   workspace: device scratch of at least dq8_qgemm_workspace_bytes(), may be
 *      NULL when that is 0.
 * M == 0, N == 0 launch nothing and succeed; K == 0 yields epilogue(0). */
int dq8_qgemm(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw,
              void* out, int64_t ldo, int64_t M, int64_t N, int64_t K, int tp_a,
              int tp_b, int epilogue, const void* bias, int bias_kind,
              const float* sx, int64_t n_sx, const float* sw, int64_t n_sw,
              const float* so, int64_t n_so, int32_t zx, int32_t zw, int32_t zo,
              void* workspace, size_t workspace_bytes, void* stream);

/* A quantized linear on a few rows of f32 activations in ONE launch:
 *   xq  = dq8_quantize(X; scale sx[0], zero point 0, [-128, 127], round_mode)
 *   out = dq8_qgemm(xq, W [N,K], ..., epilogue, ...)                       bit for bit,
 * the fused mhlo_disc.quantize in front of quantized_dot_general (R disc/transforms/
 * disc_lower_quantize_and_dequantize.cc:77-94 emits the quantize as elementwise ops that the
 * compiler's fusion then merges with neighbours; here it is merged into the GEMM): the
 * activations are quantized on their way into the matrix cores and the int8 tensor is never
 * written.  X: device f32 [M,K], row stride ldx floats; W: device int8 [N,K], row stride ldw;
 * sx: one device f32 (also the GEMM's input scale); epilogues, bias, sw, so, zo as for
 * dq8_qgemm (all but REQUANT_FIXEDPOINT; with REQUANT_*_DEQUANT_F32 the whole
 * quantize -> linear -> dequantize chain is one launch).  Every workgroup along N quantizes
 * its rows again, so this pays only for M <= dq8_qlinear_f32_fused_max_rows(N, K) (0 when
 * K % 16 != 0); more rows are an error: run the two operators.  Rows of X and W 16-byte
 * aligned. */
int64_t dq8_qlinear_f32_fused_max_rows(int64_t N, int64_t K);
int dq8_qlinear_f32(const float* X, int64_t ldx, const int8_t* W, int64_t ldw, void* out,
                    int64_t ldo, int64_t M, int64_t N, int64_t K, int epilogue, const void* bias,
                    int bias_kind, const float* sx, const float* sw, int64_t n_sw,
                    const float* so, int64_t n_so, int32_t zo, int round_mode, void* stream);

/* Operators the compiler fuses behind a quantized GEMM or convolution (its elementwise
 * fusion around quantized_dot_general / quantized_conv, next to the graph rewrites of
 * R disc/transforms/disc_quantized_dot_merge.cc:155-456): done in the producing kernel's
 * epilogue, bit for bit what the separate operators give.  With q the int8 result of the
 * requantisation stage (output scale so[0], zero point zo):
 *   table     out = table[(uint8_t) q]: any dequantize -> activation -> quantize chain
 *             (256 device bytes, as for dq8_lut8); int8 out, no residual
 *   residual  t = (float)(q - zo) * so[0] + r(m, n)        [dq8_dequantize, then an f32 add]
 *             r = residual[m, n] (DQ8_RESIDUAL_F32) or
 *                 (float)(residual[m, n] - residual_zp) * residual_scale[0] (DQ8_RESIDUAL_S8)
 *             relu: t = t < 0 ? 0 : t
 *             out_scale given: out = sat8(rne(t / out_scale[0] + out_zp))   [dq8_quantize]
 *             (epilogues REQUANT_CPU / REQUANT_GPU / REQUANT_FIXEDPOINT, int8 out);
 *             out_scale NULL: out = t (epilogues REQUANT_*_DEQUANT_F32, f32 out)
 * The residual is [M, N] with row stride ldr elements (a convolution's: the layout of its
 * output).  Scales are device pointers. */
#define DQ8_RESIDUAL_NONE 0
#define DQ8_RESIDUAL_F32 1
#define DQ8_RESIDUAL_S8 2
typedef struct dq8_postops {
  const void* residual;
  int residual_kind;
  int64_t ldr;
  const float* residual_scale;
  int32_t residual_zp;
  int relu;
  const float* out_scale;
  int32_t out_zp;
  const void* table;
} dq8_postops_t;

/* dq8_qgemm with operators fused behind it (post may be NULL: then it is dq8_qgemm). */
int dq8_qgemm_fused(const int8_t* A, int64_t lda, const int8_t* W, int64_t ldw, void* out,
                    int64_t ldo, int64_t M, int64_t N, int64_t K, int tp_a, int tp_b,
                    int epilogue, const void* bias, int bias_kind, const float* sx,
                    int64_t n_sx, const float* sw, int64_t n_sw, const float* so, int64_t n_so,
                    int32_t zx, int32_t zw, int32_t zo, void* workspace, size_t workspace_bytes,
                    const dq8_postops_t* post, void* stream);

/* Name of the kernel configuration dq8_qgemm chooses on the current device for dense,
 * 16-byte aligned, k-contiguous operands of this shape without zero points or fused operators
 * and an output element of `out_bytes` bytes (1: int8, 4: int32 / f32), e.g.
 * "pipe_256x256x128_w8"; "" for an empty or oversized problem.  For logs and profiles (the
 * counterpart of the algorithm the reference prints with DISC_GPU_ENABLE_PROFILE,
 * R ral/context/stream_executor_based_impl.cc:427-483); the returned string is static. */
const char* dq8_qgemm_kernel_name(int64_t M, int64_t N, int64_t K, int out_bytes);

/* dst[c, r] = src[r, c] for an int8 matrix src [rows, cols] with row stride ld;
 * dst is dense [cols, rows].  Used to put [K,N] weights into the kernels' [N,K]
 * layout once (the reference's counterpart is oneDNN's weight pre-packing,
 * R ral/context/common_context_impl_quantization.cc:1365-1383). */
int dq8_transpose_s8(const int8_t* src, int64_t ld, int8_t* dst, int64_t rows,
                     int64_t cols, void* stream);

/* ---- weight-only quantized GEMM ----------------------------------------- */

/* out[m,n] = (sum_k x[m,k] * (w(n,k) - zero_points[n])) * scale[n] + bias[n]: floating-point
 * activations times 8-bit weights with a per-output-channel scale and zero point, i.e.
 * matmul(x, dequantize(w)^T) + bias.  Replaces the target of the reference's
 * `ral_pdll_weight_only_qgemm` custom call
 * (R pytorch_blade/tests/disc/pdl/pdll_files/gpu/weight_only_qgemm.pdll:2-104, operands
 * input, weight, [bias,] weight_scale, weight_zero_point; the layout pass that marks the
 * weight as reordered is R tao_compiler/mlir/disc/transforms/
 * disc_transform_weight_data_layout_for_weight_only_gemm.cc:305).
 * x, out, scale, bias: x_dtype (DQ8_DTYPE_*), rows ldx / ldo elements apart; bias and
 * zero_points may be NULL; w: uint8 (w_signed = 0) or int8 (1), [N,K] with rows ldw bytes
 * apart if tp_b, else [K,N] as the custom call passes it.  Zero points must lie in
 * [-1024, 1024] for uint8 weights and in [-1152, 896] for int8 weights (the kernels subtract
 * the half 1024 + zp, + 128 for int8, which holds integers exactly only up to 2048; they are
 * device data and not checked).  [K,N] weights are transposed into `workspace`
 * (dq8_weight_only_qgemm_workspace_bytes) on every call; a runtime does that once per constant
 * weight with dq8_transpose_s8 and passes tp_b = 1.  Without the scratch, or with K % 16 != 0
 * or rows that are not 16-byte aligned, a slower kernel without alignment rules runs.
 * Accumulation is f32; f32 activations enter the matrix cores as two halves: about 22
 * significant bits for |x| >= 1/8, an absolute 2^-25 per activation below (the low half is then
 * a subnormal half), and |x| must stay below 65504. */
size_t dq8_weight_only_qgemm_workspace_bytes(int64_t N, int64_t K, int tp_b);
/* The scratch that lets the call also split the k range over several workgroups per tile when
 * M is too small for the tiles to fill the chip (f32 partial sums and a
 * reduction launch behind the GEMM; the sums of the k ranges are added in their order, so the
 * result does not depend on timing).  Includes the bytes of the function above; with less the
 * call still runs, unsplit. */
size_t dq8_weight_only_qgemm_workspace_bytes_ex(int64_t M, int64_t N, int64_t K, int tp_b,
                                                int x_dtype);
int dq8_weight_only_qgemm(const void* x, int x_dtype, int64_t ldx, const void* w, int w_signed,
                          int64_t ldw, int tp_b, const void* scale, const int32_t* zero_points,
                          const void* bias, void* out, int64_t ldo, int64_t M, int64_t N,
                          int64_t K, void* workspace, size_t workspace_bytes, void* stream);

/* The compiler's constant-weight layout, undone.  The reference's pipeline rewrites every
 * rank-2 ui8 *constant* weight [K,N] of a `ral_pdll_weight_only_qgemm` call with a byte
 * permutation meant for NVIDIA tensor-core fragments and sets `weight_should_be_reordered =
 * false` (R tao_compiler/mlir/disc/transforms/
 * disc_transform_weight_data_layout_for_weight_only_gemm.cc:54-300, composed at :362-370, run
 * from R tao_compiler/mlir/disc/disc_compiler.cc:257-258).  This puts such a buffer
 * (`reordered`, K*N bytes) back in order, as the dense [N,K] matrix dq8_weight_only_qgemm takes
 * with tp_b = 1 (`w_nk`, K*N bytes, must not overlap).  The pass is a permutation only for
 * K % 64 == 0 and N % 4 == 0 (elsewhere it indexes out of bounds); other shapes are refused.
 * Both buffers 16-byte aligned.  A runtime does this once per constant. */
int dq8_weight_only_undo_compiler_layout(const uint8_t* reordered, uint8_t* w_nk, int64_t K,
                                         int64_t N, void* stream);

/* ---- int8 convolution (rank 4) ---------------------------------------- */

/* Implicit-GEMM convolution.  Layouts are described exactly as ral_qconv's
 * metadata vector describes them (17 host int32: input {batch,channel,h,w} dim
 * indices, kernel {in,out,h,w}, output {batch,channel,h,w}, strides[2],
 * dilations[2], weight_is_const) with host padding {top,bottom,left,right}.
 * The MFMA path takes NHWC x OHWI -> NHWC with Ci % 16 == 0; every other layout
 * runs the generic kernel.  Epilogue/bias/scales as for dq8_qgemm with N = Co. */
int dq8_qconv2d(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                const int64_t w_sizes[4], const int32_t padding[4],
                const int32_t metadata[17], void* out,
                const int64_t out_sizes[4], int epilogue, const void* bias,
                int bias_kind, const float* sx, const float* sw, int64_t n_sw,
                const float* so, int32_t zo, void* stream);
/* The same with device scratch: NHWC x OHWI with Ci % 16 != 0 (an RGB first layer) then
 * stays on the MFMA path -- input and weights are rewritten into `workspace`
 * (256-byte aligned, dq8_qconv2d_workspace_bytes() bytes) with the channels zero-filled
 * to the next multiple of 16.  With less scratch the result is the same, from the
 * generic kernel.  dq8_qconv2d_workspace_bytes() is 0 when nothing would be rewritten. */
size_t dq8_qconv2d_workspace_bytes(const int64_t in_sizes[4], const int64_t w_sizes[4],
                                   const int32_t metadata[17]);
/* The same with the result's sizes: additionally covers NCHW x OIHW -> NCHW convolutions, whose
 * tensors are re-laid out as NHWC / OHWI in the scratch so that they run on the MFMA kernels
 * (what the reference's GPU path does around its NHWC int8 kernels,
 * R ral/context/stream_executor_based_impl.cc:1073-1112); without the scratch they take the
 * generic kernel. */
size_t dq8_qconv2d_workspace_bytes_ex(const int64_t in_sizes[4], const int64_t w_sizes[4],
                                      const int64_t out_sizes[4], const int32_t metadata[17]);
int dq8_qconv2d_ws(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                   const int64_t w_sizes[4], const int32_t padding[4],
                   const int32_t metadata[17], void* out, const int64_t out_sizes[4],
                   int epilogue, const void* bias, int bias_kind, const float* sx,
                   const float* sw, int64_t n_sw, const float* so, int32_t zo,
                   void* workspace, size_t workspace_bytes, void* stream);
/* dq8_qconv2d_ws with operators fused behind it (post may be NULL). */
int dq8_qconv2d_fused(const int8_t* in, const int64_t in_sizes[4], const int8_t* w,
                      const int64_t w_sizes[4], const int32_t padding[4],
                      const int32_t metadata[17], void* out, const int64_t out_sizes[4],
                      int epilogue, const void* bias, int bias_kind, const float* sx,
                      const float* sw, int64_t n_sw, const float* so, int32_t zo,
                      void* workspace, size_t workspace_bytes, const dq8_postops_t* post,
                      void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DISC_Q8_H_ */
