// RAL entries of the quantized-inference hot path for the gpu device, backed by the
// hand-written gfx950 kernels (include/disc_q8.h).
//
// Entries and the reference functions they replace (R = tao_compiler/mlir/ral/):
//   ral_qgemm                   R context/stream_executor_based_impl.cc:427-483 (per
//                               tensor, gpu) and the per-channel signature of
//                               R context/common_context_impl_quantization.cc:1196-1266
//   ral_pdll_qgemm              R context/quantized_gpu_kernel_impl.cc:329-461 (gpu
//                               signatures: int8 / f32 bias already in output units)
//                               and the CPU-style signatures of
//                               R context/common_context_impl_quantization.cc:1268-1672
//                               (f32 / s32 / no bias, per-channel weight scale)
//   ral_pdll_qgemm_per_channel  R context/quantized_gpu_kernel_impl.cc:197-321
//   ral_qconv                   R context/stream_executor_based_impl.cc:1831-1948
//   ral_pdll_qconv2d            R context/common_context_impl_quantization.cc:352-607
//                               (registered there for cpu only, :1685; same signature
//                               and attributes here for gpu)
//   ral_quantize / ral_dequantize
//                               no runtime symbol in the reference: its compiler
//                               expands mhlo_disc.quantize / dequantize into loops
//                               (disc/transforms/disc_lower_quantize_and_dequantize.cc);
//                               these entries run the same arithmetic as one kernel.
//
// Differences from the reference that callers can observe:
//   * scales stay on the device: nothing here copies them to the host or
//     synchronises the stream (the reference does both on the first or on every
//     call); the kernels read the scale buffers themselves.
//   * ral_qconv applies the per-channel weight scale to every channel (the
//     reference reads element 0 only).
//   * errors are reported through Context::signalError and the entry returns; no
//     kernel is launched after an error.
//   * DISC_GPU_ENABLE_PROFILE=1 (or "true") makes the GEMM and convolution entries time
//     their kernels with a pair of events, wait for them, and log the fields the reference
//     prints under DISC_CPU_ENABLE_PROFILE (R context/common_context_impl.cc:66-73, 116-119;
//     R context/common_context_impl_quantization.cc:722-743): operand pointers, m / n / k,
//     "Math Ops", "Bytes", bandwidth and rate.  Off by default; on, every call blocks.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>

#include "disc_q8.h"
#include "mlir/ral/context/base/hip/hip_context_impl.h"
#include "mlir/ral/context/context_util.h"
#include "mlir/ral/context/conv_attr_util.h"
#include "mlir/ral/context/pdll_util.h"
#include "mlir/ral/device/gpu/gpu_driver.h"
#include "mlir/ral/ral_context.h"
#include "mlir/ral/ral_helper.h"
#include "mlir/ral/ral_logging.h"

namespace tao {
namespace ral {
namespace gpu {
namespace q8 {

namespace {

void fail(ExecutionContext* ctx, const std::string& what) {
  ctx->signalError(Context::FAILURE, what);
}

// Reports a kernel-library failure; returns true when `status` was an error.
bool kernelFailed(ExecutionContext* ctx, int status, const char* who) {
  if (status == 0) return false;
  fail(ctx, std::string(who) + ": " + dq8_last_error());
  return true;
}

bool initProfileMode() {
  const char* env = std::getenv("DISC_GPU_ENABLE_PROFILE");
  if (!env) return false;
  std::string v = env;
  std::transform(v.begin(), v.end(), v.begin(),
                 [](unsigned char c) { return (char)std::tolower(c); });
  return v == "true" || v == "1";
}

bool isProfilingEnabled() {
  static bool enabled = initProfileMode();
  return enabled;
}

// Times what is put on `stream` between construction and stop() (profile mode only;
// stop() waits for the stream).  Event failures switch the timer off rather than
// failing the call.
class StreamTimer {
 public:
  explicit StreamTimer(void* stream) : stream_(static_cast<hipStream_t>(stream)) {
    if (!isProfilingEnabled()) return;
    if (hipEventCreate(&begin_) != hipSuccess) return;
    if (hipEventCreate(&end_) != hipSuccess) {
      (void)hipEventDestroy(begin_);
      return;
    }
    on_ = hipEventRecord(begin_, stream_) == hipSuccess;
  }
  ~StreamTimer() {
    if (begin_) (void)hipEventDestroy(begin_);
    if (end_) (void)hipEventDestroy(end_);
    (void)hipGetLastError();
  }
  bool on() const { return on_; }
  // nanoseconds since construction, or a negative value
  double stop() {
    float ms = -1.0f;
    if (!on_ || hipEventRecord(end_, stream_) != hipSuccess ||
        hipEventSynchronize(end_) != hipSuccess ||
        hipEventElapsedTime(&ms, begin_, end_) != hipSuccess)
      return -1.0;
    return (double)ms * 1e6;
  }

 private:
  hipStream_t stream_;
  hipEvent_t begin_ = nullptr, end_ = nullptr;
  bool on_ = false;
};

// Which output stage the entries use whose signature the reference implements twice on the
// CPU -- with oneDNN's float post-ops on x86 and with Arm Compute Library's fixed-point
// multiplier and shift on AArch64 (ral_qgemm with per-channel weight scales, ral_qconv,
// ral_pdll_qconv2d: R context/common_context_impl_quantization.cc:1680-1696 against
// :1699-1719).  Default: the float stage; DISC_GPU_REQUANT_FIXEDPOINT=1 selects the integer
// one, for results identical to the reference's AArch64 build.
// (Read at every call, like the reference reads its DISC_* switches at the point of use: a
// host may run graphs of both kinds in one process.)
int sharedSignatureStage() {
  const char* v = std::getenv("DISC_GPU_REQUANT_FIXEDPOINT");
  return v && *v && std::strcmp(v, "0") != 0 && std::strcmp(v, "false") != 0
             ? DQ8_EPI_REQUANT_FIXEDPOINT
             : DQ8_EPI_REQUANT_CPU;
}

GPUDriver* driverOf(ExecutionContext* ctx) {
  auto* d = ctx->getDriver<GPUDriver>(GPUDriver::name());
  if (!d) fail(ctx, "GPUDriver not found");
  return d;
}

// [K,N] constant weights are turned into the kernels' [N,K] layout once and kept
// for the life of the context, keyed by the weight buffer's address and shape.
struct PackedWeightState : public Context::Resource {
  // how the bytes at `ptr` are laid out: plain [K,N], or [K,N] after the compiler's
  // weight-only layout pass
  enum Layout { kPlainKN = 0, kCompilerReorderedKN = 1 };
  struct Key {
    const void* ptr;
    int64_t k, n;
    int layout = kPlainKN;
    bool operator==(const Key& o) const {
      return ptr == o.ptr && k == o.k && n == o.n && layout == o.layout;
    }
  };
  struct Hash {
    size_t operator()(const Key& k) const {
      return std::hash<const void*>()(k.ptr) ^ (std::hash<int64_t>()(k.k) * 1000003u) ^
             (std::hash<int64_t>()(k.n) * 998244353u) ^ (size_t)k.layout;
    }
  };
  std::mutex mu;
  std::unordered_map<Key, int8_t*, Hash> packed;
};

const char* kPackedWeightState = "tao_ral.gpu.qgemm_packed_weight_i8";

struct GemmOperands {
  const int8_t* a = nullptr;
  const int8_t* w = nullptr;
  int64_t m = 0, n = 0, k = 0;
  bool tp_a = false, tp_b = false;
  bool weight_is_const = false;
  int32_t zx = 0, zw = 0;   // input / weight zero point: acc = sum (a - zx)(w - zw)
};

struct Epilogue {
  int mode = DQ8_EPI_REQUANT_CPU;
  const void* bias = nullptr;
  int bias_kind = DQ8_BIAS_NONE;
  const float* sx = nullptr;
  const float* sw = nullptr;
  const float* so = nullptr;
  int64_t n_sx = 1, n_sw = 1, n_so = 1;
  int32_t zo = 0;
};

// Launches the GEMM, providing scratch (or the cached packed weight) for
// operands that are not k-contiguous.
void runGemm(ExecutionContext* ctx, void* stream_handle, GemmOperands op, const Epilogue& e,
             void* out, const char* who, const dq8_postops_t* post = nullptr) {
  GPUDriver* drv = driverOf(ctx);
  if (!drv) return;
  void* stream = drv->asCUStream(ctx, stream_handle);

  if (!op.tp_b && op.weight_is_const && op.k > 0) {
    auto* state = ctx->getOrCreateResource<PackedWeightState>(
        kPackedWeightState, [] { return new PackedWeightState; });
    if (!state) return;
    std::lock_guard<std::mutex> guard(state->mu);
    PackedWeightState::Key key{op.w, op.k, op.n};
    auto it = state->packed.find(key);
    if (it == state->packed.end()) {
      auto* nk = static_cast<int8_t*>(drv->alloc_persistent(ctx, (size_t)(op.n * op.k)));
      if (!nk) return;
      // [K,N] -> [N,K], once; ordered before the GEMM on the same stream
      if (kernelFailed(ctx, dq8_transpose_s8(op.w, op.n, nk, op.k, op.n, stream), who)) return;
      it = state->packed.emplace(key, nk).first;
    }
    op.w = it->second;
    op.tp_b = true;
  }

  const int64_t lda = op.tp_a ? op.m : op.k;
  const int64_t ldw = op.tp_b ? op.k : op.n;
  // (with a zero point: room for the correction vectors that keep the problem on the MFMA
  // kernels)
  const size_t ws_bytes =
      dq8_qgemm_workspace_bytes_zp(op.m, op.n, op.k, op.tp_a, op.tp_b, op.zx, op.zw);
  void* ws = nullptr;
  if (ws_bytes) {
    ws = drv->alloc(ctx, ws_bytes);
    if (!ws) return;
  }
  StreamTimer timer(stream);
  int st = dq8_qgemm_fused(op.a, lda, op.w, ldw, out, op.n, op.m, op.n, op.k, op.tp_a, op.tp_b,
                           e.mode, e.bias, e.bias_kind, e.sx, e.n_sx, e.sw, e.n_sw, e.so, e.n_so,
                           op.zx, op.zw, e.zo, ws, ws_bytes, post, stream);
  if (timer.on() && st == 0) {
    const double ns = timer.stop();
    const int64_t bytes = op.m * op.k + op.k * op.n + op.m * op.n;
    TAO_LOG(INFO) << who << " (gpu):\n"
                << "\tpa = " << (const void*)op.a << "\n"
                << "\tpb = " << (const void*)op.w << "\n"
                << "\tpc = " << (const void*)out << "\n"
                << "\tm = " << op.m << "\n"
                << "\tn = " << op.n << "\n"
                << "\tk = " << op.k << "\n"
                << "\ttp_a = " << op.tp_a << "\n"
                << "\ttp_b = " << op.tp_b << "\n"
                << "\tweight_is_const = " << op.weight_is_const << "\n"
                << "\tMath Ops = " << 2 * op.m * op.n * op.k << "\n"
                << "\tBytes = " << bytes << "\n"
                << "\tElapsed = " << ns / 1e3 << " us\n"
                << "\tBandwidth = " << double(bytes) / ns << " GB\n"
                << "\tGOPS = " << double(2 * op.m * op.n * op.k) / ns << "\n";
  }
  // the pool hands `ws` out again only to later work on the same stream, which is
  // ordered after this launch
  if (ws) drv->dealloc(ctx, ws);
  kernelFailed(ctx, st, who);
}

// The profile record of a convolution (the reference's dumpConvLikeKernelProflingInfo,
// R context/common_context_impl_mkldnn.h:605): sizes, work and rates.
void logConvProfile(const char* who, const int64_t in[4], const int64_t w[4], const int64_t out[4],
                    double ns) {
  int64_t out_elems = 1, in_elems = 1, w_elems = 1;
  for (int i = 0; i < 4; ++i) {
    out_elems *= out[i];
    in_elems *= in[i];
    w_elems *= w[i];
  }
  // every output element takes (filter elements per output channel) multiply-adds
  const int64_t per_out = w[0] > 0 ? w_elems / w[0] : 0;
  const int64_t ops = 2 * out_elems * per_out;
  const int64_t bytes = in_elems + w_elems + out_elems;
  TAO_LOG(INFO) << who << " (gpu):\n"
              << "\tinput = " << in[0] << "x" << in[1] << "x" << in[2] << "x" << in[3] << "\n"
              << "\tkernel = " << w[0] << "x" << w[1] << "x" << w[2] << "x" << w[3] << "\n"
              << "\toutput = " << out[0] << "x" << out[1] << "x" << out[2] << "x" << out[3] << "\n"
              << "\tMath Ops = " << ops << "\n"
              << "\tBytes = " << bytes << "\n"
              << "\tElapsed = " << ns / 1e3 << " us\n"
              << "\tBandwidth = " << double(bytes) / ns << " GB\n"
              << "\tGOPS = " << double(ops) / ns << "\n";
}

template <typename T, int N>
bool requireContiguous(ExecutionContext* ctx, const MemRefType<T, N>& m, const char* who,
                       const char* what) {
  if (isContiguous(m)) return true;
  fail(ctx, std::string(who) + ": " + what + " must be a dense row-major memref");
  return false;
}

}  // namespace

// ------------------------------------------------------------------ ral_qgemm
// result = sat8(rne(((s_x * s_w[n]) / s_o) * acc)); zero points are not read (the
// reference gpu entry does not read them either).
template <int WS_RANK>
void ral_qgemm_impl(ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, 2> input,
                    MemRefType<int8_t, 2> weight, MemRefType<float, 0> inputScales,
                    MemRefType<float, WS_RANK> weightScales, MemRefType<float, 0> resultScales,
                    MemRefType<int8_t, 2> result, bool tp_a, bool tp_b, bool weight_is_const) {
  static const char* who = "ral_qgemm";
  if (isEmptyMemref(input) || isEmptyMemref(weight) || isEmptyMemref(result)) {
    TAO_VLOG(1) << "ral_qgemm: early return for empty tensor";
    return;
  }
  GemmOperands op;
  op.m = tp_a ? input.sizes[1] : input.sizes[0];
  op.k = tp_a ? input.sizes[0] : input.sizes[1];
  op.n = tp_b ? weight.sizes[0] : weight.sizes[1];
  if (op.k != (tp_b ? weight.sizes[1] : weight.sizes[0])) {
    fail(ctx, "mismatch contraction dim for ral_qgemm");
    return;
  }
  if (result.sizes[0] != op.m || result.sizes[1] != op.n) {
    fail(ctx, "ral_qgemm: result shape does not match the operands");
    return;
  }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, weight, who, "weight") ||
      !requireContiguous(ctx, result, who, "result"))
    return;
  op.a = input.data;
  op.w = weight.data;
  op.tp_a = tp_a;
  op.tp_b = tp_b;
  op.weight_is_const = weight_is_const;
  Epilogue e;
  e.mode = WS_RANK == 1 ? sharedSignatureStage() : DQ8_EPI_REQUANT_CPU;
  e.sx = inputScales.data;
  e.sw = weightScales.data;
  e.so = resultScales.data;
  if constexpr (WS_RANK == 1) {
    e.n_sw = weightScales.sizes[0];
    if (e.n_sw != 1 && e.n_sw != op.n) {
      fail(ctx, "ral_qgemm: weight scale must have 1 or N entries");
      return;
    }
  }
  runGemm(ctx, stream_handle, op, e, result.data, who);
}

void ral_qgemm(ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, 2> input,
               MemRefType<int8_t, 2> weight, MemRefType<float, 0> inputScales,
               MemRefType<int32_t, 0> /*inputZeroPoints*/, MemRefType<float, 0> weightScales,
               MemRefType<int32_t, 0> /*weightZeroPoints*/, MemRefType<float, 0> resultScales,
               MemRefType<int32_t, 0> /*resultZeroPoints*/, MemRefType<int8_t, 2> result,
               bool tp_a, bool tp_b, bool weight_is_const) {
  ral_qgemm_impl<0>(ctx, stream_handle, input, weight, inputScales, weightScales, resultScales,
                    result, tp_a, tp_b, weight_is_const);
}

void ral_qgemm_per_channel(ExecutionContext* ctx, void* stream_handle,
                           MemRefType<int8_t, 2> input, MemRefType<int8_t, 2> weight,
                           MemRefType<float, 0> inputScales,
                           MemRefType<int32_t, 0> /*inputZeroPoints*/,
                           MemRefType<float, 1> weightScales,
                           MemRefType<int32_t, 1> /*weightZeroPoints*/,
                           MemRefType<float, 0> resultScales,
                           MemRefType<int32_t, 0> /*resultZeroPoints*/,
                           MemRefType<int8_t, 2> result, bool tp_a, bool tp_b,
                           bool weight_is_const) {
  ral_qgemm_impl<1>(ctx, stream_handle, input, weight, inputScales, weightScales, resultScales,
                    result, tp_a, tp_b, weight_is_const);
}

// ------------------------------------------------------------- ral_pdll_qgemm
namespace {

// Flattens the leading dims of a rank-N input into M and allocates the result
// through the driver.  Returns false (with `result` describing a null buffer of
// the right shape) when there is nothing to compute.
template <int N, typename InT = int8_t, typename OutT = int8_t>
bool prepareResult(ExecutionContext* ctx, const MemRefType<InT, N>& input, int64_t n,
                   int64_t* m, MemRefType<OutT, N>* result) {
  int64_t sizes[N];
  *m = 1;
  for (int i = 0; i < N - 1; ++i) {
    *m *= input.sizes[i];
    sizes[i] = input.sizes[i];
  }
  sizes[N - 1] = n;
  if (*m == 0 || n == 0) {
    *result = assignMemRef<OutT, N>(nullptr, sizes);
    return false;
  }
  GPUDriver* drv = driverOf(ctx);
  if (!drv) {
    *result = assignMemRef<OutT, N>(nullptr, sizes);
    return false;
  }
  void* data = drv->alloc(ctx, (size_t)(*m * n) * sizeof(OutT));
  *result = assignMemRef<OutT, N>(data, sizes);
  return data != nullptr;
}

// Zero points of ral_pdll_* calls are host-resident ("s" placement in the PDLL
// patterns).  The entries with the reference's gpu signatures are symmetric, as the
// reference's are (its gpu kernels never read the zero points).
bool symmetricOrFail(ExecutionContext* ctx, const int32_t* zx, int64_t n_zx, const int32_t* zw,
                     int64_t n_zw, const char* who) {
  for (int64_t i = 0; i < n_zx; ++i)
    if (zx && zx[i] != 0) {
      fail(ctx, std::string(who) + ": non-zero input zero point is not supported");
      return false;
    }
  for (int64_t i = 0; i < n_zw; ++i)
    if (zw && zw[i] != 0) {
      fail(ctx, std::string(who) + ": non-zero weight zero point is not supported");
      return false;
    }
  return true;
}

}  // namespace

// GPU signatures: weight [N,K], bias already in output-quantised units,
// out = sat8(rne(((s_x*s_w)/s_o) * acc + bias[n])).
template <int N, typename BiasT>
MemRefType<int8_t, N> ral_pdll_qgemm_gpu(ExecutionContext* ctx, void* stream_handle,
                                         MemRefType<int8_t, N> input,
                                         MemRefType<int8_t, 2> weight,
                                         MemRefType<BiasT, 1> bias,
                                         MemRefType<float, 0> inputScales,
                                         MemRefType<int32_t, 0> inputZeroPoints,
                                         MemRefType<float, 0> weightScales,
                                         MemRefType<int32_t, 0> weightZeroPoints,
                                         MemRefType<float, 0> resultScales,
                                         MemRefType<int32_t, 0> resultZeroPoints,
                                         void* /*customAttrs*/) {
  static const char* who = "ral_pdll_qgemm";
  GemmOperands op;
  op.n = weight.sizes[0];
  op.k = weight.sizes[1];
  MemRefType<int8_t, N> result;
  if (input.sizes[N - 1] != op.k && !isEmptyMemref(input)) {
    fail(ctx, "mismatch contraction dim for ral_pdll_qgemm");
    int64_t zeros[N] = {0};
    return assignMemRef<int8_t, N>(nullptr, zeros);
  }
  if (!prepareResult<N>(ctx, input, op.n, &op.m, &result)) return result;
  if (!symmetricOrFail(ctx, inputZeroPoints.data, 1, weightZeroPoints.data, 1, who) ||
      (resultZeroPoints.data && resultZeroPoints.data[0] != 0 &&
       (fail(ctx, "ral_pdll_qgemm: non-zero result zero point is not supported"), true)))
    return result;
  if (bias.sizes[0] != op.n) {
    fail(ctx, "ral_pdll_qgemm: bias must have N entries");
    return result;
  }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, weight, who, "weight"))
    return result;
  op.a = input.data;
  op.w = weight.data;
  op.tp_b = true;
  Epilogue e;
  e.mode = DQ8_EPI_REQUANT_GPU;
  e.bias = bias.data;
  e.bias_kind = std::is_same<BiasT, float>::value ? DQ8_BIAS_F32 : DQ8_BIAS_S8;
  e.sx = inputScales.data;
  e.sw = weightScales.data;
  e.so = resultScales.data;
  runGemm(ctx, stream_handle, op, e, result.data, who);
  return result;
}

// Merged-QKV form: all three scales are [N] vectors, int8 bias.
template <int N>
MemRefType<int8_t, N> ral_pdll_qgemm_per_channel(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<int8_t, 1> bias, MemRefType<float, 1> inputScales,
    MemRefType<int32_t, 1> inputZeroPoints, MemRefType<float, 1> weightScales,
    MemRefType<int32_t, 1> weightZeroPoints, MemRefType<float, 1> resultScales,
    MemRefType<int32_t, 1> resultZeroPoints, void* /*customAttrs*/) {
  static const char* who = "ral_pdll_qgemm_per_channel";
  GemmOperands op;
  op.n = weight.sizes[0];
  op.k = weight.sizes[1];
  MemRefType<int8_t, N> result;
  if (input.sizes[N - 1] != op.k && !isEmptyMemref(input)) {
    fail(ctx, "mismatch contraction dim for ral_pdll_qgemm_per_channel");
    int64_t zeros[N] = {0};
    return assignMemRef<int8_t, N>(nullptr, zeros);
  }
  if (!prepareResult<N>(ctx, input, op.n, &op.m, &result)) return result;
  if (inputScales.sizes[0] != op.n || weightScales.sizes[0] != op.n ||
      resultScales.sizes[0] != op.n || bias.sizes[0] != op.n) {
    fail(ctx, "ral_pdll_qgemm_per_channel: scales and bias must have N entries");
    return result;
  }
  if (!symmetricOrFail(ctx, inputZeroPoints.data, inputZeroPoints.sizes[0],
                       weightZeroPoints.data, weightZeroPoints.sizes[0], who))
    return result;
  for (int64_t i = 0; resultZeroPoints.data && i < resultZeroPoints.sizes[0]; ++i)
    if (resultZeroPoints.data[i] != 0) {
      fail(ctx, "ral_pdll_qgemm_per_channel: non-zero result zero point is not supported");
      return result;
    }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, weight, who, "weight"))
    return result;
  op.a = input.data;
  op.w = weight.data;
  op.tp_b = true;
  Epilogue e;
  e.mode = DQ8_EPI_REQUANT_GPU;
  e.bias = bias.data;
  e.bias_kind = DQ8_BIAS_S8;
  e.sx = inputScales.data;
  e.sw = weightScales.data;
  e.so = resultScales.data;
  e.n_sx = e.n_sw = e.n_so = op.n;
  runGemm(ctx, stream_handle, op, e, result.data, who);
  return result;
}

// CPU-style signatures on the gpu device: per-channel weight scale, bias f32 /
// s32 / none, weight [K,N] unless the `transpose_b` attr says otherwise,
// out = sat8(rne((f32(acc) + b32[n]) * ((s_x*s_w[n])/s_o) + z_o)).
namespace {

struct NoBias {};

// What a fused entry adds behind the requantisation (ral_pdll_qgemm_fused below).
struct FusedTail {
  const float* residual = nullptr;   // f32, the result's shape; null = none
  int64_t residual_elems = 0;
  const uint8_t* table = nullptr;    // 256 entries; null = none
};

template <int N, typename OutT = int8_t>
MemRefType<OutT, N> pdllQgemmCpuStyle(ExecutionContext* ctx, void* stream_handle,
                                      MemRefType<int8_t, N> input,
                                      MemRefType<int8_t, 2> weight, const void* bias,
                                      int64_t n_bias, int bias_kind,
                                      MemRefType<float, 0> inputScales,
                                      MemRefType<int32_t, 0> inputZeroPoints,
                                      MemRefType<float, 1> weightScales,
                                      MemRefType<int32_t, 1> weightZeroPoints,
                                      MemRefType<float, 0> resultScales,
                                      MemRefType<int32_t, 0> resultZeroPoints,
                                      void* customAttrs, int stage = DQ8_EPI_REQUANT_CPU,
                                      const FusedTail* tail = nullptr) {
  static const char* who = "ral_pdll_qgemm";
  int64_t zeros[N] = {0};
  MemRefType<OutT, N> result = assignMemRef<OutT, N>(nullptr, zeros);
  bool relu = false;
  bool tp_a = false, tp_b = false, weight_is_const = false;
  if (customAttrs) {
    PDLAttr* attr = getOrParsePDLAttr(ctx, customAttrs, "ral_pdll_qgemm_gpu_cpu_style");
    if (!attr || attr->getType() != "dict") {
      fail(ctx, "fail to parse custom_attrs\n");
      return result;
    }
    auto& dict = attr->as<DictPDLAttr>();
    auto flag = [&](const char* key) {
      return dict.hasKey(key) && dict.get(key).getType() == "bool" &&
             dict.get(key).as<BoolPDLAttr>().getValue();
    };
    tp_a = flag("transpose_a");
    tp_b = flag("transpose_b");
    weight_is_const = flag("weight_is_const");
    relu = flag("relu");
  }
  if (tp_a) {
    fail(ctx, "ral_pdll_qgemm: transpose_a is not supported on gpu");
    return result;
  }
  GemmOperands op;
  op.k = tp_b ? weight.sizes[1] : weight.sizes[0];
  op.n = tp_b ? weight.sizes[0] : weight.sizes[1];
  if (input.sizes[N - 1] != op.k && !isEmptyMemref(input)) {
    fail(ctx, "mismatch contraction dim for ral_pdll_qgemm");
    return result;
  }
  if (!prepareResult<N, int8_t, OutT>(ctx, input, op.n, &op.m, &result)) return result;
  // One input zero point and one weight zero point, as oneDNN takes them from the
  // reference's CPU entries (ideep matmul.hpp:516-517, 548-549; the reference silently uses
  // element 0 of a weight zero-point vector -- a vector that is not uniform is refused here).
  op.zx = inputZeroPoints.data ? inputZeroPoints.data[0] : 0;
  op.zw = weightZeroPoints.data && weightZeroPoints.sizes[0] > 0 ? weightZeroPoints.data[0] : 0;
  for (int64_t i = 1; weightZeroPoints.data && i < weightZeroPoints.sizes[0]; ++i)
    if (weightZeroPoints.data[i] != op.zw) {
      fail(ctx, "ral_pdll_qgemm: per-channel weight zero points are not supported");
      return result;
    }
  if (weightScales.sizes[0] != 1 && weightScales.sizes[0] != op.n) {
    fail(ctx, "ral_pdll_qgemm: weight scale must have 1 or N entries");
    return result;
  }
  if (bias_kind != DQ8_BIAS_NONE && n_bias != op.n) {
    fail(ctx, "ral_pdll_qgemm: bias must have N entries");
    return result;
  }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, weight, who, "weight"))
    return result;
  op.a = input.data;
  op.w = weight.data;
  op.tp_b = tp_b;
  op.weight_is_const = weight_is_const;
  Epilogue e;
  e.mode = stage;
  e.bias = bias;
  e.bias_kind = bias_kind;
  e.sx = inputScales.data;
  e.sw = weightScales.data;
  e.n_sw = weightScales.sizes[0];
  e.so = resultScales.data;
  e.zo = resultZeroPoints.data ? resultZeroPoints.data[0] : 0;
  dq8_postops_t post = {};
  if (tail) {
    if (tail->residual) {
      if (tail->residual_elems != op.m * op.n) {
        fail(ctx, "ral_pdll_qgemm_fused: the residual must have the result's shape");
        return result;
      }
      post.residual = tail->residual;
      post.residual_kind = DQ8_RESIDUAL_F32;
      post.ldr = op.n;
      post.relu = relu ? 1 : 0;
    }
    post.table = tail->table;
  }
  runGemm(ctx, stream_handle, op, e, result.data, who, tail ? &post : nullptr);
  return result;
}

}  // namespace

// ---- ral_pdll_qgemm_fused: operators the compiler's elementwise fusion leaves next to a
// quantized GEMM, taken into the call.  No counterpart among the reference's entries (there the
// fused elementwise kernel is generated code next to the custom call); a pattern set for this
// runtime rewrites  dequantize(ral_pdll_qgemm(...))  [+ residual, relu]  or
// quantize(f(dequantize(ral_pdll_qgemm(...))))  into one of these.  Operands up to
// customAttrs are those of the CPU-style ral_pdll_qgemm with an f32 bias
// (R context/common_context_impl_quantization.cc:1268-1423); the results are bit for bit what
// the separate operators give.
//   (..., attrs)                   -> f32   dequantize of the int8 result, in the epilogue
//   (..., residual f32, attrs)     -> f32   the same + residual [, relu per attr `relu`]
//   (..., table ui8[256], attrs)   -> int8  table[(uint8) q]: any dequantize -> f -> quantize
template <int N>
MemRefType<float, N> ral_pdll_qgemm_fused_dequant(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<float, 1> bias, MemRefType<float, 0> inputScales,
    MemRefType<int32_t, 0> inputZeroPoints, MemRefType<float, 1> weightScales,
    MemRefType<int32_t, 1> weightZeroPoints, MemRefType<float, 0> resultScales,
    MemRefType<int32_t, 0> resultZeroPoints, void* customAttrs) {
  return pdllQgemmCpuStyle<N, float>(ctx, stream_handle, input, weight, bias.data, bias.sizes[0],
                                     DQ8_BIAS_F32, inputScales, inputZeroPoints, weightScales,
                                     weightZeroPoints, resultScales, resultZeroPoints, customAttrs,
                                     DQ8_EPI_REQUANT_CPU_DEQUANT_F32);
}

template <int N>
MemRefType<float, N> ral_pdll_qgemm_fused_dequant_residual(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<float, 1> bias, MemRefType<float, 0> inputScales,
    MemRefType<int32_t, 0> inputZeroPoints, MemRefType<float, 1> weightScales,
    MemRefType<int32_t, 1> weightZeroPoints, MemRefType<float, 0> resultScales,
    MemRefType<int32_t, 0> resultZeroPoints, MemRefType<float, N> residual, void* customAttrs) {
  int64_t zeros[N] = {0};
  if (!isContiguous(residual)) {
    ctx->signalError(Context::FAILURE, "ral_pdll_qgemm_fused: residual must be a dense memref");
    return assignMemRef<float, N>(nullptr, zeros);
  }
  FusedTail tail;
  tail.residual = residual.data;
  tail.residual_elems = 1;
  for (int i = 0; i < N; ++i) tail.residual_elems *= residual.sizes[i];
  return pdllQgemmCpuStyle<N, float>(ctx, stream_handle, input, weight, bias.data, bias.sizes[0],
                                     DQ8_BIAS_F32, inputScales, inputZeroPoints, weightScales,
                                     weightZeroPoints, resultScales, resultZeroPoints, customAttrs,
                                     DQ8_EPI_REQUANT_CPU_DEQUANT_F32, &tail);
}

template <int N>
MemRefType<int8_t, N> ral_pdll_qgemm_fused_table(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<float, 1> bias, MemRefType<float, 0> inputScales,
    MemRefType<int32_t, 0> inputZeroPoints, MemRefType<float, 1> weightScales,
    MemRefType<int32_t, 1> weightZeroPoints, MemRefType<float, 0> resultScales,
    MemRefType<int32_t, 0> resultZeroPoints, MemRefType<uint8_t, 1> table, void* customAttrs) {
  int64_t zeros[N] = {0};
  if (table.sizes[0] != 256 || !table.data) {
    ctx->signalError(Context::FAILURE, "ral_pdll_qgemm_fused: the table must have 256 entries");
    return assignMemRef<int8_t, N>(nullptr, zeros);
  }
  FusedTail tail;
  tail.table = table.data;
  return pdllQgemmCpuStyle<N, int8_t>(ctx, stream_handle, input, weight, bias.data, bias.sizes[0],
                                      DQ8_BIAS_F32, inputScales, inputZeroPoints, weightScales,
                                      weightZeroPoints, resultScales, resultZeroPoints, customAttrs,
                                      DQ8_EPI_REQUANT_CPU, &tail);
}

// ---- ral_pdll_qlinear: quantize -> ral_pdll_qgemm -> dequantize on f32 activations, the whole
// quantized linear as one call (no counterpart among the reference's entries; a pattern set for
// this runtime rewrites the chain the reference's patterns leave,  dequantize(ral_pdll_qgemm(
// quantize(x), ...)),  into it).  Operands: those of the CPU-style ral_pdll_qgemm with an f32
// bias, the input f32; the input is quantized with inputScales, zero point 0 (others are
// refused), to int8, rounding per attr `round_mode` (0 half away from zero, 1 half to even,
// default 1).  A few rows run as one launch (dq8_qlinear_f32); more as quantize + GEMM with the
// int8 activations in pool scratch.  Bit for bit the three operators' result.
template <int N>
MemRefType<float, N> ral_pdll_qlinear(
    ExecutionContext* ctx, void* stream_handle, MemRefType<float, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<float, 1> bias, MemRefType<float, 0> inputScales,
    MemRefType<int32_t, 0> inputZeroPoints, MemRefType<float, 1> weightScales,
    MemRefType<int32_t, 1> weightZeroPoints, MemRefType<float, 0> resultScales,
    MemRefType<int32_t, 0> resultZeroPoints, void* customAttrs) {
  static const char* who = "ral_pdll_qlinear";
  int64_t zeros[N] = {0};
  MemRefType<float, N> result = assignMemRef<float, N>(nullptr, zeros);
  bool tp_b = false, weight_is_const = false;
  int round_mode = DQ8_ROUND_HALF_TO_EVEN;
  if (customAttrs) {
    PDLAttr* attr = getOrParsePDLAttr(ctx, customAttrs, who);
    if (!attr || attr->getType() != "dict") {
      fail(ctx, "fail to parse custom_attrs\n");
      return result;
    }
    auto& dict = attr->as<DictPDLAttr>();
    auto flag = [&](const char* key) {
      return dict.hasKey(key) && dict.get(key).getType() == "bool" &&
             dict.get(key).as<BoolPDLAttr>().getValue();
    };
    if (flag("transpose_a")) {
      fail(ctx, std::string(who) + ": transpose_a is not supported on gpu");
      return result;
    }
    tp_b = flag("transpose_b");
    weight_is_const = flag("weight_is_const");
    if (dict.hasKey("round_mode") && dict.get("round_mode").getType() == "int")
      round_mode = (int)dict.get("round_mode").as<IntPDLAttr>().getValue();
  }
  if ((inputZeroPoints.data && inputZeroPoints.data[0] != 0)) {
    fail(ctx, std::string(who) + ": a non-zero input zero point is not supported; run "
                                 "ral_quantize and ral_pdll_qgemm");
    return result;
  }
  for (int64_t i = 0; weightZeroPoints.data && i < weightZeroPoints.sizes[0]; ++i)
    if (weightZeroPoints.data[i] != 0) {
      fail(ctx, std::string(who) + ": non-zero weight zero points are not supported; run "
                                   "ral_quantize and ral_pdll_qgemm");
      return result;
    }
  const int64_t k = tp_b ? weight.sizes[1] : weight.sizes[0];
  const int64_t n = tp_b ? weight.sizes[0] : weight.sizes[1];
  if (input.sizes[N - 1] != k && !isEmptyMemref(input)) {
    fail(ctx, std::string(who) + ": mismatch contraction dim");
    return result;
  }
  if ((weightScales.sizes[0] != 1 && weightScales.sizes[0] != n) || bias.sizes[0] != n) {
    fail(ctx, std::string(who) + ": weight scale must have 1 or N entries, bias N");
    return result;
  }
  int64_t m = 0;
  if (!prepareResult<N, float, float>(ctx, input, n, &m, &result)) return result;
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, weight, who, "weight"))
    return result;
  GPUDriver* drv = driverOf(ctx);
  if (!drv) return result;
  void* stream = drv->asCUStream(ctx, stream_handle);
  const int32_t zo = resultZeroPoints.data ? resultZeroPoints.data[0] : 0;
  // one launch: a few rows against [N,K] weights
  if (tp_b && k > 0 && m <= dq8_qlinear_f32_fused_max_rows(n, k) &&
      reinterpret_cast<uintptr_t>(input.data) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(weight.data) % 16 == 0) {
    kernelFailed(ctx,
                 dq8_qlinear_f32(input.data, k, weight.data, k, result.data, n, m, n, k,
                                 DQ8_EPI_REQUANT_CPU_DEQUANT_F32, bias.data, DQ8_BIAS_F32,
                                 inputScales.data, weightScales.data, weightScales.sizes[0],
                                 resultScales.data, 1, zo, round_mode, stream),
                 who);
    return result;
  }
  // quantize into pool scratch (the zero point 0 it needs on the device sits behind the data)
  const size_t xq_bytes = ((size_t)(m * k) + 255) / 256 * 256;
  auto* xq = static_cast<int8_t*>(drv->alloc(ctx, xq_bytes + 256));
  if (!xq) return result;
  int32_t* zero_zp = reinterpret_cast<int32_t*>(xq + xq_bytes);
  if (kernelFailed(ctx, dq8_fill(zero_zp, 0, 4, stream), who) ||
      kernelFailed(ctx,
                   dq8_quantize(input.data, xq, DQ8_I8, 1, 1, m * k, inputScales.data, zero_zp, 1,
                                -128, 127, round_mode, stream),
                   who)) {
    drv->dealloc(ctx, xq);
    return result;
  }
  GemmOperands op;
  op.a = xq;
  op.w = weight.data;
  op.m = m;
  op.n = n;
  op.k = k;
  op.tp_b = tp_b;
  op.weight_is_const = weight_is_const;
  Epilogue e;
  e.mode = DQ8_EPI_REQUANT_CPU_DEQUANT_F32;
  e.bias = bias.data;
  e.bias_kind = DQ8_BIAS_F32;
  e.sx = inputScales.data;
  e.sw = weightScales.data;
  e.n_sw = weightScales.sizes[0];
  e.so = resultScales.data;
  e.zo = zo;
  runGemm(ctx, stream_handle, op, e, result.data, who);
  drv->dealloc(ctx, xq);   // (later work on the stream is ordered behind the GEMM)
  return result;
}

template <int N>
MemRefType<int8_t, N> ral_pdll_qgemm_s8_s8_s8_f32_per_channel(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<float, 1> bias, MemRefType<float, 0> inputScales,
    MemRefType<int32_t, 0> inputZeroPoints, MemRefType<float, 1> weightScales,
    MemRefType<int32_t, 1> weightZeroPoints, MemRefType<float, 0> resultScales,
    MemRefType<int32_t, 0> resultZeroPoints, void* customAttrs) {
  return pdllQgemmCpuStyle<N>(ctx, stream_handle, input, weight, bias.data, bias.sizes[0],
                              DQ8_BIAS_F32, inputScales, inputZeroPoints, weightScales,
                              weightZeroPoints, resultScales, resultZeroPoints, customAttrs);
}

template <int N>
MemRefType<int8_t, N> ral_pdll_qgemm_s8_s8_s8_s32_per_channel(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<int32_t, 1> bias,
    MemRefType<float, 0> inputScales, MemRefType<int32_t, 0> inputZeroPoints,
    MemRefType<float, 1> weightScales, MemRefType<int32_t, 1> weightZeroPoints,
    MemRefType<float, 0> resultScales, MemRefType<int32_t, 0> resultZeroPoints,
    void* customAttrs) {
  return pdllQgemmCpuStyle<N>(ctx, stream_handle, input, weight, bias.data, bias.sizes[0],
                              DQ8_BIAS_S32, inputScales, inputZeroPoints, weightScales,
                              weightZeroPoints, resultScales, resultZeroPoints, customAttrs);
}

template <int N>
MemRefType<int8_t, N> ral_pdll_qgemm_s8_s8_s8_per_channel(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<float, 0> inputScales,
    MemRefType<int32_t, 0> inputZeroPoints, MemRefType<float, 1> weightScales,
    MemRefType<int32_t, 1> weightZeroPoints, MemRefType<float, 0> resultScales,
    MemRefType<int32_t, 0> resultZeroPoints, void* customAttrs) {
  return pdllQgemmCpuStyle<N>(ctx, stream_handle, input, weight, nullptr, 0, DQ8_BIAS_NONE,
                              inputScales, inputZeroPoints, weightScales, weightZeroPoints,
                              resultScales, resultZeroPoints, customAttrs);
}

// The per-tensor signatures of ral_pdll_qgemm: in the reference they exist only in the
// AArch64 build, on Arm Compute Library's fixed-point output stage
// (ral_pdll_qgemm_acl_s8_s8_s8_per_tensor<2,3,4> and ..._s32_per_tensor<2,3>,
// R context/common_context_impl_quantization.cc:747-1187, registered :1689-1695):
//   out = clamp8(stage(acc + bias[n]; multiplier = (s_x s_w) / s_o) + z_o)
// Mirrored here for device "gpu" with the same stage, so that a graph rewritten with the
// AArch64 pattern set gives the AArch64 results.
namespace {
MemRefType<float, 1> asVector(const MemRefType<float, 0>& m) {
  MemRefType<float, 1> v;
  v.basePtr = m.basePtr;
  v.data = m.data;
  v.offset = m.offset;
  v.sizes[0] = 1;
  v.strides[0] = 1;
  return v;
}
MemRefType<int32_t, 1> asVector(const MemRefType<int32_t, 0>& m) {
  MemRefType<int32_t, 1> v;
  v.basePtr = m.basePtr;
  v.data = m.data;
  v.offset = m.offset;
  v.sizes[0] = 1;
  v.strides[0] = 1;
  return v;
}
}  // namespace

template <int N>
MemRefType<int8_t, N> ral_pdll_qgemm_s8_s8_s8_per_tensor(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<float, 0> inputScales,
    MemRefType<int32_t, 0> inputZeroPoints, MemRefType<float, 0> weightScales,
    MemRefType<int32_t, 0> weightZeroPoints, MemRefType<float, 0> resultScales,
    MemRefType<int32_t, 0> resultZeroPoints, void* customAttrs) {
  return pdllQgemmCpuStyle<N>(ctx, stream_handle, input, weight, nullptr, 0, DQ8_BIAS_NONE,
                              inputScales, inputZeroPoints, asVector(weightScales),
                              asVector(weightZeroPoints), resultScales, resultZeroPoints,
                              customAttrs, DQ8_EPI_REQUANT_FIXEDPOINT);
}

template <int N>
MemRefType<int8_t, N> ral_pdll_qgemm_s8_s8_s8_s32_per_tensor(
    ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, N> input,
    MemRefType<int8_t, 2> weight, MemRefType<int32_t, 1> bias,
    MemRefType<float, 0> inputScales, MemRefType<int32_t, 0> inputZeroPoints,
    MemRefType<float, 0> weightScales, MemRefType<int32_t, 0> weightZeroPoints,
    MemRefType<float, 0> resultScales, MemRefType<int32_t, 0> resultZeroPoints,
    void* customAttrs) {
  return pdllQgemmCpuStyle<N>(ctx, stream_handle, input, weight, bias.data, bias.sizes[0],
                              DQ8_BIAS_S32, inputScales, inputZeroPoints, asVector(weightScales),
                              asVector(weightZeroPoints), resultScales, resultZeroPoints,
                              customAttrs, DQ8_EPI_REQUANT_FIXEDPOINT);
}

// ------------------------------------------------------------------ ral_qconv
// out = sat8(rne(((s_x*s_w[co])/s_o) * conv_s32(in, w))); padding and metadata are
// host memrefs; zero points are not read.
// ---- ral_pdll_weight_only_qgemm -------------------------------------------------------
// Target of the reference's weight-only patterns (R pytorch_blade/tests/disc/pdl/pdll_files/
// gpu/weight_only_qgemm.pdll:2-104; placements "d,d,d,d" and "d,d,d,d,d"): activations f32 or
// f16 [..., K], weight ui8 [K, N] (the pattern transposes the [N, K] constant), [bias [N],]
// per-channel scale [N] and zero point [N], all on the device; result [..., N] in the
// activation type.  The reference tree has no implementation of this entry to compare with.
// custom_attrs: `weight_should_be_reordered`.
//  * false: the compiler's layout pass (R tao_compiler/mlir/disc/transforms/
//    disc_transform_weight_data_layout_for_weight_only_gemm.cc:305-410, run unconditionally from
//    R tao_compiler/mlir/disc/disc_compiler.cc:257-258) has matched, i.e. the weight is a rank-2
//    ui8 *constant* (:322-338) whose bytes it has permuted for NVIDIA tensor-core fragments
//    (:362-370).  The permutation is undone once per weight buffer into the kernels' [N,K]
//    layout and kept for the life of the context (the buffer is a constant by construction).
//  * true (what the pattern emits and the pass leaves when it does not match): the weight is
//    plain [K,N] and may be the result of another operator (the reference's test IR feeds it
//    from an mhlo.transpose), whose buffer the allocator reuses for other contents.  The
//    [N,K] copy is therefore cached only for buffers known to outlive executions (constants
//    served by ral_const); any other weight is transposed on every call, into pool scratch.
namespace {

template <typename T>
struct WoDtype;
template <>
struct WoDtype<float> {
  static constexpr int value = DQ8_DTYPE_F32;
};
template <>
struct WoDtype<float16> {
  static constexpr int value = DQ8_DTYPE_F16;
};

template <typename T, int N>
MemRefType<T, N> weightOnlyQgemm(ExecutionContext* ctx, void* stream_handle,
                                 MemRefType<T, N> input, MemRefType<uint8_t, 2> weight,
                                 const T* bias, int64_t n_bias, MemRefType<T, 1> scales,
                                 MemRefType<int32_t, 1> zeroPoints, void* customAttrs) {
  static const char* who = "ral_pdll_weight_only_qgemm";
  int64_t sizes[N] = {0};
  MemRefType<T, N> result = assignMemRef<T, N>(nullptr, sizes);
  bool reordered_by_compiler = false;
  if (customAttrs) {
    PDLAttr* attr = getOrParsePDLAttr(ctx, customAttrs, who);
    if (!attr || attr->getType() != "dict") {
      fail(ctx, "fail to parse custom_attrs\n");
      return result;
    }
    auto& dict = attr->as<DictPDLAttr>();
    reordered_by_compiler = dict.hasKey("weight_should_be_reordered") &&
                            dict.get("weight_should_be_reordered").getType() == "bool" &&
                            !dict.get("weight_should_be_reordered").as<BoolPDLAttr>().getValue();
  }
  const int64_t k = weight.sizes[0], n = weight.sizes[1];
  if (reordered_by_compiler && (k % 64 != 0 || n % 4 != 0)) {
    // (the pass indexes out of bounds there; what it leaves is not a permutation of the weight)
    fail(ctx, std::string(who) + ": weight_should_be_reordered = false needs K % 64 == 0 and "
                                 "N % 4 == 0, the shapes the compiler's layout pass is defined for");
    return result;
  }
  if (input.sizes[N - 1] != k && !isEmptyMemref(input)) {
    fail(ctx, std::string(who) + ": mismatch contraction dim");
    return result;
  }
  if (scales.sizes[0] != n || zeroPoints.sizes[0] != n || (bias && n_bias != n)) {
    fail(ctx, std::string(who) + ": scale, zero point and bias must have N entries");
    return result;
  }
  int64_t m = 1;
  for (int i = 0; i < N - 1; ++i) {
    m *= input.sizes[i];
    sizes[i] = input.sizes[i];
  }
  sizes[N - 1] = n;
  result = assignMemRef<T, N>(nullptr, sizes);
  if (m == 0 || n == 0) return result;
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, weight, who, "weight"))
    return result;
  GPUDriver* drv = driverOf(ctx);
  if (!drv) return result;
  void* stream = drv->asCUStream(ctx, stream_handle);
  // The kernels' [N,K] layout, cached per weight buffer where the buffer is known to be a
  // constant; a [K,N] weight that is not goes through scratch on every call.
  const uint8_t* w_nk = nullptr;
  const bool cacheable =
      k > 0 && (reordered_by_compiler || gpu::isPersistentDeviceBuffer(ctx, weight.data));
  if (cacheable) {
    auto* state = ctx->getOrCreateResource<PackedWeightState>(
        kPackedWeightState, [] { return new PackedWeightState; });
    if (!state) return result;
    std::lock_guard<std::mutex> guard(state->mu);
    PackedWeightState::Key key{weight.data, k, n,
                               reordered_by_compiler ? PackedWeightState::kCompilerReorderedKN
                                                     : PackedWeightState::kPlainKN};
    auto it = state->packed.find(key);
    if (it == state->packed.end()) {
      auto* nk = static_cast<int8_t*>(drv->alloc_persistent(ctx, (size_t)(n * k)));
      if (!nk) return result;
      const int st =
          reordered_by_compiler
              ? dq8_weight_only_undo_compiler_layout(weight.data, reinterpret_cast<uint8_t*>(nk), k,
                                                     n, stream)
              : dq8_transpose_s8(reinterpret_cast<const int8_t*>(weight.data), n, nk, k, n, stream);
      if (kernelFailed(ctx, st, who)) return result;
      it = state->packed.emplace(key, nk).first;
    }
    w_nk = reinterpret_cast<const uint8_t*>(it->second);
  }
  const int tp_b = w_nk ? 1 : 0;
  void* data = drv->alloc(ctx, (size_t)(m * n) * sizeof(T));
  if (!data) return result;
  result = assignMemRef<T, N>(data, sizes);
  // (scratch for the transposed copy of a weight that is not cached and for the partial sums of
  // a launch split over k when m is small; handed back to the pool right after the launch,
  // which later work on the same stream is ordered behind)
  size_t ws_bytes = dq8_weight_only_qgemm_workspace_bytes_ex(m, n, k, tp_b, WoDtype<T>::value);
  void* ws = ws_bytes ? drv->alloc(ctx, ws_bytes) : nullptr;
  if (!ws) ws_bytes = 0;                                   // (the call then runs unsplit)
  StreamTimer timer(stream);
  const int st = dq8_weight_only_qgemm(input.data, WoDtype<T>::value, k,
                                       w_nk ? static_cast<const void*>(w_nk) : weight.data, 0,
                                       tp_b ? k : n, tp_b, scales.data, zeroPoints.data, bias, data,
                                       n, m, n, k, ws, ws_bytes, stream);
  if (ws) drv->dealloc(ctx, ws);
  if (timer.on() && st == 0) {
    const double ns = timer.stop();
    const int64_t bytes = (m * k + m * n) * (int64_t)sizeof(T) + k * n;
    TAO_LOG(INFO) << who << " (gpu):\n"
                  << "\tm = " << m << "\n"
                  << "\tn = " << n << "\n"
                  << "\tk = " << k << "\n"
                  << "\tweight = "
                  << (reordered_by_compiler ? "compiler layout, cached"
                                            : (w_nk ? "[K,N] constant, cached" : "[K,N], per call"))
                  << "\n"
                  << "\tMath Ops = " << 2 * m * n * k << "\n"
                  << "\tBytes = " << bytes << "\n"
                  << "\tElapsed = " << ns / 1e3 << " us\n"
                  << "\tBandwidth = " << double(bytes) / ns << " GB\n"
                  << "\tGFLOPS = " << double(2 * m * n * k) / ns << "\n";
  }
  kernelFailed(ctx, st, who);
  return result;
}

}  // namespace

template <typename T, int N>
MemRefType<T, N> ral_pdll_weight_only_qgemm(ExecutionContext* ctx, void* stream_handle,
                                            MemRefType<T, N> input,
                                            MemRefType<uint8_t, 2> weight,
                                            MemRefType<T, 1> scales,
                                            MemRefType<int32_t, 1> zeroPoints,
                                            void* customAttrs) {
  return weightOnlyQgemm<T, N>(ctx, stream_handle, input, weight, nullptr, 0, scales, zeroPoints,
                               customAttrs);
}

template <typename T, int N>
MemRefType<T, N> ral_pdll_weight_only_qgemm_bias(ExecutionContext* ctx, void* stream_handle,
                                                 MemRefType<T, N> input,
                                                 MemRefType<uint8_t, 2> weight,
                                                 MemRefType<T, 1> bias, MemRefType<T, 1> scales,
                                                 MemRefType<int32_t, 1> zeroPoints,
                                                 void* customAttrs) {
  return weightOnlyQgemm<T, N>(ctx, stream_handle, input, weight, bias.data, bias.sizes[0], scales,
                               zeroPoints, customAttrs);
}

void ral_qconv(ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, 4> input,
               MemRefType<int8_t, 4> kernel, MemRefType<int32_t, 1> padding,
               MemRefType<float, 0> inputScales, MemRefType<int32_t, 0> /*inputZeroPoints*/,
               MemRefType<float, 1> weightScales, MemRefType<int32_t, 1> /*weightZeroPoints*/,
               MemRefType<float, 0> resultScales, MemRefType<int32_t, 0> /*resultZeroPoints*/,
               MemRefType<int8_t, 4> output, MemRefType<int32_t, 1> metadata) {
  static const char* who = "ral_qconv";
  if (isEmptyMemref(input) || isEmptyMemref(kernel) || isEmptyMemref(output)) {
    TAO_VLOG(1) << "ral_qconv: early return for empty tensor";
    return;
  }
  if (padding.sizes[0] != 4 || metadata.sizes[0] != 17) {
    fail(ctx, "ral_qconv: rank-4 convolution needs 4 padding and 17 metadata entries");
    return;
  }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, kernel, who, "kernel") ||
      !requireContiguous(ctx, output, who, "output"))
    return;
  GPUDriver* drv = driverOf(ctx);
  if (!drv) return;
  void* stream = drv->asCUStream(ctx, stream_handle);
  // (scratch for channel counts that are not a multiple of 16 and for the NHWC copies of
  // NCHW tensors; handed back to the pool
  // right after the launch, which later work on the same stream is ordered behind)
  const size_t ws_bytes =
      dq8_qconv2d_workspace_bytes_ex(input.sizes, kernel.sizes, output.sizes, metadata.data);
  void* ws = ws_bytes ? drv->alloc(ctx, ws_bytes) : nullptr;
  if (ws_bytes && !ws) return;
  StreamTimer timer(stream);
  int st = dq8_qconv2d_ws(input.data, input.sizes, kernel.data, kernel.sizes, padding.data,
                          metadata.data, output.data, output.sizes, sharedSignatureStage(),
                          nullptr, DQ8_BIAS_NONE, inputScales.data, weightScales.data,
                          weightScales.sizes[0], resultScales.data, 0, ws, ws_bytes, stream);
  if (ws) drv->dealloc(ctx, ws);
  if (timer.on() && st == 0) {
    // the output-channel extent first, as logConvProfile expects
    const int ko = metadata.data[5];
    int64_t w[4] = {kernel.sizes[ko], 1, 1, 1};
    for (int i = 0, j = 1; i < 4; ++i)
      if (i != ko) w[j++] = kernel.sizes[i];
    logConvProfile(who, input.sizes, w, output.sizes, timer.stop());
  }
  kernelFailed(ctx, st, who);
}

// The older entry without zero-point operands (R context/common_context_impl_quantization.cc:
// 38-44, registered at :1680 as "ral_qconv_s8_s8_s8"): the same convolution.
void ral_qconv_s8_s8_s8(ExecutionContext* ctx, void* stream_handle, MemRefType<int8_t, 4> input,
                        MemRefType<int8_t, 4> kernel, MemRefType<int32_t, 1> padding,
                        MemRefType<float, 0> inputScales, MemRefType<float, 1> filterScales,
                        MemRefType<float, 0> outputScales, MemRefType<int8_t, 4> output,
                        MemRefType<int32_t, 1> metadata) {
  MemRefType<int32_t, 0> no_zp0 = assignMemRef_0d<int32_t>(nullptr);
  int64_t zero[1] = {0};
  MemRefType<int32_t, 1> no_zp1 = assignMemRef<int32_t, 1>(nullptr, zero);
  ral_qconv(ctx, stream_handle, input, kernel, padding, inputScales, no_zp0, filterScales, no_zp1,
            outputScales, no_zp0, output, metadata);
}

// ----------------------------------------------------------- ral_pdll_qconv2d
// The attribute-driven convolution entry: data_format / strides / dilations / padding
// come as custom attributes, the result is allocated here.  Weights are
// [out_channels, filter_h, filter_w, in_channels].
//   out = sat8(rne(f32(conv_s32(in, w)) * ((s_x*s_w[co])/s_o) + z_o))
MemRefType<int8_t, 4> ral_pdll_qconv2d(ExecutionContext* ctx, void* stream_handle,
                                       MemRefType<int8_t, 4> input,
                                       MemRefType<int8_t, 4> weight,
                                       MemRefType<float, 0> inputScales,
                                       MemRefType<int32_t, 0> inputZeroPoints,
                                       MemRefType<float, 1> weightScales,
                                       MemRefType<int32_t, 1> weightZeroPoints,
                                       MemRefType<float, 0> resultScales,
                                       MemRefType<int32_t, 0> resultZeroPoints,
                                       void* customAttrs) {
  static const char* who = "ral_pdll_qconv2d";
  int64_t zeros[4] = {0, 0, 0, 0};
  MemRefType<int8_t, 4> result = assignMemRef<int8_t, 4>(nullptr, zeros);
  if (isEmptyMemref(input) || isEmptyMemref(weight)) {
    TAO_VLOG(1) << who << ": early return for empty tensor";
    return result;
  }
  PDLAttr* attr = customAttrs ? getOrParsePDLAttr(ctx, customAttrs, who) : nullptr;
  if (!attr || attr->getType() != "dict") {
    fail(ctx, "fail to parse custom_attrs\n");
    return result;
  }
  auto& dict = attr->as<DictPDLAttr>();
  auto has = [&](const char* key, const char* type) {
    return dict.hasKey(key) && dict.get(key).getType() == type;
  };
  if (!has("data_format", "str") || !has("padding", "str") || !has("strides", "intArray") ||
      !has("dilations", "intArray")) {
    fail(ctx, std::string(who) + ": data_format, padding, strides and dilations are required");
    return result;
  }
  std::vector<int64_t> explicit_paddings;
  if (has("explicit_paddings", "intArray"))
    explicit_paddings = dict.get("explicit_paddings").as<IntArrayPDLAttr>().getValue();
  const bool weight_is_const = has("weight_is_const", "bool") &&
                               dict.get("weight_is_const").as<BoolPDLAttr>().getValue();
  Conv2dPlan plan;
  const std::string err =
      planConv2d(dict.get("data_format").as<StrPDLAttr>().getValue(),
                 dict.get("strides").as<IntArrayPDLAttr>().getValue(),
                 dict.get("dilations").as<IntArrayPDLAttr>().getValue(),
                 dict.get("padding").as<StrPDLAttr>().getValue(), explicit_paddings,
                 weight_is_const, input.sizes, weight.sizes, &plan);
  if (!err.empty()) {
    fail(ctx, std::string(who) + ": " + err);
    return result;
  }
  if (!symmetricOrFail(ctx, inputZeroPoints.data, 1, weightZeroPoints.data,
                       weightZeroPoints.sizes[0], who))
    return result;
  if (weightScales.sizes[0] != 1 && weightScales.sizes[0] != weight.sizes[0]) {
    fail(ctx, std::string(who) + ": weight scale must have 1 or out_channels entries");
    return result;
  }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, weight, who, "weight"))
    return result;
  int64_t total = 1;
  for (int i = 0; i < 4; ++i) {
    if (plan.result_sizes[i] < 0) plan.result_sizes[i] = 0;
    total *= plan.result_sizes[i];
  }
  GPUDriver* drv = driverOf(ctx);
  if (!drv) return result;
  if (total == 0) return assignMemRef<int8_t, 4>(nullptr, plan.result_sizes);
  auto* data = static_cast<int8_t*>(drv->alloc(ctx, (size_t)total));
  if (!data) return result;
  result = assignMemRef<int8_t, 4>(data, plan.result_sizes);
  void* stream = drv->asCUStream(ctx, stream_handle);
  const int32_t zo = resultZeroPoints.data ? resultZeroPoints.data[0] : 0;
  const size_t ws_bytes = dq8_qconv2d_workspace_bytes_ex(input.sizes, weight.sizes,
                                                         plan.result_sizes, plan.metadata);
  void* ws = ws_bytes ? drv->alloc(ctx, ws_bytes) : nullptr;
  if (ws_bytes && !ws) return result;
  StreamTimer timer(stream);
  int st = dq8_qconv2d_ws(input.data, input.sizes, weight.data, weight.sizes, plan.padding,
                          plan.metadata, result.data, result.sizes, sharedSignatureStage(),
                          nullptr, DQ8_BIAS_NONE, inputScales.data, weightScales.data,
                          weightScales.sizes[0], resultScales.data, zo, ws, ws_bytes, stream);
  if (ws) drv->dealloc(ctx, ws);
  if (timer.on() && st == 0)   // weights are [out_channels, h, w, in_channels] here
    logConvProfile(who, input.sizes, weight.sizes, result.sizes, timer.stop());
  kernelFailed(ctx, st, who);
  return result;
}

// ------------------------------------------------- ral_quantize / ral_dequantize
// axis < 0 means per tensor (rank-0 scale / zero point); otherwise the scale and
// zero point vectors run along dimension `axis`.  Scale and zero point are device
// buffers.
namespace {

template <int N>
void view3(const int64_t (&sizes)[N], int64_t axis, int64_t* outer, int64_t* nch,
           int64_t* inner) {
  *outer = *nch = *inner = 1;
  if (axis < 0) {
    for (int i = 0; i < N; ++i) *inner *= sizes[i];
    return;
  }
  for (int i = 0; i < N; ++i) {
    if (i < axis) *outer *= sizes[i];
    else if (i == axis) *nch = sizes[i];
    else *inner *= sizes[i];
  }
}

}  // namespace

template <typename QT>
struct QuantKind;
template <> struct QuantKind<int8_t> { static constexpr int value = DQ8_I8; };
template <> struct QuantKind<uint8_t> { static constexpr int value = DQ8_U8; };
template <> struct QuantKind<int16_t> { static constexpr int value = DQ8_I16; };
template <> struct QuantKind<uint16_t> { static constexpr int value = DQ8_U16; };
template <> struct QuantKind<int32_t> { static constexpr int value = DQ8_I32; };
template <> struct QuantKind<uint32_t> { static constexpr int value = DQ8_U32; };

template <typename QT, int N, int SR>
void ral_quantize(ExecutionContext* ctx, void* stream_handle, MemRefType<float, N> input,
                  MemRefType<float, SR> scale, MemRefType<int32_t, SR> zeroPoint,
                  MemRefType<QT, N> result, int64_t axis, int64_t quantMin, int64_t quantMax,
                  int64_t roundMode) {
  static const char* who = "ral_quantize";
  if (isEmptyMemref(input)) return;
  for (int i = 0; i < N; ++i)
    if (input.sizes[i] != result.sizes[i]) {
      fail(ctx, "ral_quantize: result shape differs from the input's");
      return;
    }
  if ((SR == 0) != (axis < 0) || axis >= N) {
    fail(ctx, "ral_quantize: axis does not match the rank of scale/zero_point");
    return;
  }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, result, who, "result"))
    return;
  int64_t outer, nch, inner;
  view3<N>(input.sizes, axis, &outer, &nch, &inner);
  int64_t n_q = 1;
  if constexpr (SR == 1) {
    n_q = scale.sizes[0];
    if (n_q != nch || zeroPoint.sizes[0] != nch) {
      fail(ctx, "ral_quantize: scale/zero_point length differs from the axis extent");
      return;
    }
  }
  GPUDriver* drv = driverOf(ctx);
  if (!drv) return;
  int st = dq8_quantize_ex(input.data, DQ8_DTYPE_F32, result.data, QuantKind<QT>::value, outer, nch,
                           inner, scale.data, zeroPoint.data, SR == 0 ? 1 : n_q, quantMin,
                           quantMax, (int)roundMode, drv->asCUStream(ctx, stream_handle));
  kernelFailed(ctx, st, who);
}

template <typename QT, int N, int SR>
void ral_dequantize(ExecutionContext* ctx, void* stream_handle, MemRefType<QT, N> input,
                    MemRefType<float, SR> scale, MemRefType<int32_t, SR> zeroPoint,
                    MemRefType<float, N> result, int64_t axis) {
  static const char* who = "ral_dequantize";
  if (isEmptyMemref(input)) return;
  for (int i = 0; i < N; ++i)
    if (input.sizes[i] != result.sizes[i]) {
      fail(ctx, "ral_dequantize: result shape differs from the input's");
      return;
    }
  if ((SR == 0) != (axis < 0) || axis >= N) {
    fail(ctx, "ral_dequantize: axis does not match the rank of scale/zero_point");
    return;
  }
  if (!requireContiguous(ctx, input, who, "input") ||
      !requireContiguous(ctx, result, who, "result"))
    return;
  int64_t outer, nch, inner;
  view3<N>(input.sizes, axis, &outer, &nch, &inner);
  int64_t n_q = 1;
  if constexpr (SR == 1) {
    n_q = scale.sizes[0];
    if (n_q != nch || zeroPoint.sizes[0] != nch) {
      fail(ctx, "ral_dequantize: scale/zero_point length differs from the axis extent");
      return;
    }
  }
  GPUDriver* drv = driverOf(ctx);
  if (!drv) return;
  int st = dq8_dequantize_ex(input.data, QuantKind<QT>::value, result.data, outer, nch, inner,
                             scale.data, zeroPoint.data, SR == 0 ? 1 : n_q,
                             drv->asCUStream(ctx, stream_handle));
  kernelFailed(ctx, st, who);
}

}  // namespace q8
}  // namespace gpu

// ---------------------------------------------------------------- registration
TAO_RAL_API("ral_qgemm", "gpu", gpu::q8::ral_qgemm);
TAO_RAL_API("ral_qgemm", "gpu", gpu::q8::ral_qgemm_per_channel);

TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_gpu<2, int8_t>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_gpu<3, int8_t>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_gpu<2, float>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_gpu<3, float>);
TAO_RAL_API("ral_pdll_qgemm_per_channel", "gpu", gpu::q8::ral_pdll_qgemm_per_channel<2>);
TAO_RAL_API("ral_pdll_qgemm_per_channel", "gpu", gpu::q8::ral_pdll_qgemm_per_channel<3>);

TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_f32_per_channel<2>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_f32_per_channel<3>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_f32_per_channel<4>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_s32_per_channel<2>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_s32_per_channel<3>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_s32_per_channel<4>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_per_channel<2>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_per_channel<3>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_per_channel<4>);

// the AArch64 build's per-tensor signatures (fixed-point output stage)
// (fused forms: no counterpart among the reference's entries)
TAO_RAL_API("ral_pdll_qgemm_fused", "gpu", gpu::q8::ral_pdll_qgemm_fused_dequant<2>);
TAO_RAL_API("ral_pdll_qgemm_fused", "gpu", gpu::q8::ral_pdll_qgemm_fused_dequant<3>);
TAO_RAL_API("ral_pdll_qgemm_fused", "gpu", gpu::q8::ral_pdll_qgemm_fused_dequant_residual<2>);
TAO_RAL_API("ral_pdll_qgemm_fused", "gpu", gpu::q8::ral_pdll_qgemm_fused_dequant_residual<3>);
TAO_RAL_API("ral_pdll_qgemm_fused", "gpu", gpu::q8::ral_pdll_qgemm_fused_table<2>);
TAO_RAL_API("ral_pdll_qgemm_fused", "gpu", gpu::q8::ral_pdll_qgemm_fused_table<3>);
TAO_RAL_API("ral_pdll_qlinear", "gpu", gpu::q8::ral_pdll_qlinear<2>);
TAO_RAL_API("ral_pdll_qlinear", "gpu", gpu::q8::ral_pdll_qlinear<3>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_per_tensor<2>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_per_tensor<3>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_per_tensor<4>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_s32_per_tensor<2>);
TAO_RAL_API("ral_pdll_qgemm", "gpu", gpu::q8::ral_pdll_qgemm_s8_s8_s8_s32_per_tensor<3>);

#define DQ8_REGISTER_WEIGHT_ONLY(T, N)                                                        \
  TAO_RAL_API("ral_pdll_weight_only_qgemm", "gpu", gpu::q8::ral_pdll_weight_only_qgemm<T, N>); \
  TAO_RAL_API("ral_pdll_weight_only_qgemm", "gpu", gpu::q8::ral_pdll_weight_only_qgemm_bias<T, N>);
DQ8_REGISTER_WEIGHT_ONLY(float, 2)
DQ8_REGISTER_WEIGHT_ONLY(float, 3)
DQ8_REGISTER_WEIGHT_ONLY(float16, 2)
DQ8_REGISTER_WEIGHT_ONLY(float16, 3)
#undef DQ8_REGISTER_WEIGHT_ONLY

TAO_RAL_API("ral_qconv", "gpu", gpu::q8::ral_qconv);
TAO_RAL_API("ral_qconv_s8_s8_s8", "gpu", gpu::q8::ral_qconv_s8_s8_s8);
TAO_RAL_API("ral_pdll_qconv2d", "gpu", gpu::q8::ral_pdll_qconv2d);

#define DQ8_REGISTER_QDQ(QT, N)                                              \
  TAO_RAL_API("ral_quantize", "gpu", gpu::q8::ral_quantize<QT, N, 0>);       \
  TAO_RAL_API("ral_quantize", "gpu", gpu::q8::ral_quantize<QT, N, 1>);       \
  TAO_RAL_API("ral_dequantize", "gpu", gpu::q8::ral_dequantize<QT, N, 0>);   \
  TAO_RAL_API("ral_dequantize", "gpu", gpu::q8::ral_dequantize<QT, N, 1>);
DQ8_REGISTER_QDQ(int8_t, 1)
DQ8_REGISTER_QDQ(int8_t, 2)
DQ8_REGISTER_QDQ(int8_t, 3)
DQ8_REGISTER_QDQ(int8_t, 4)
DQ8_REGISTER_QDQ(uint8_t, 1)
DQ8_REGISTER_QDQ(uint8_t, 2)
DQ8_REGISTER_QDQ(uint8_t, 3)
DQ8_REGISTER_QDQ(uint8_t, 4)
// the wider quantized types of the operator (disc-fold-quantize.mlir:137-247), ranks 1-2
DQ8_REGISTER_QDQ(int16_t, 1)
DQ8_REGISTER_QDQ(int16_t, 2)
DQ8_REGISTER_QDQ(uint16_t, 1)
DQ8_REGISTER_QDQ(uint16_t, 2)
DQ8_REGISTER_QDQ(int32_t, 1)
DQ8_REGISTER_QDQ(int32_t, 2)
DQ8_REGISTER_QDQ(uint32_t, 1)
DQ8_REGISTER_QDQ(uint32_t, 2)
#undef DQ8_REGISTER_QDQ

}  // namespace ral
}  // namespace tao
