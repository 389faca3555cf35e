// The entries a compiled program uses to talk to its surroundings: fetch its inputs,
// hand over its outputs, materialise its constants and move memrefs between host and
// device.  Counterparts in the reference:
//   ral_recv_input / ral_send_output  R context/base/base_context.cc:131-262 (device "cpu":
//                                     they are host-side calls whatever the tensor's home)
//   ral_const (gpu)                   R context/common_context_impl_cuda.cc:60-175
//   ral_const (cpu, host constants)   R context/common_context_impl.cc:279-390
//   inc_ref (reshape / bitcast)       R context/base/cuda/cuda_context_impl.cc:517-681
//   h2d / d2h / d2d on memrefs        R context/common_context_impl_cuda.cc:380-437
#include <cstring>
#include <numeric>
#include <string>
#include <vector>

#include "mlir/ral/context/base/hip/hip_context_impl.h"
#include "mlir/ral/context/context_util.h"
#include "mlir/ral/device/gpu/gpu_driver.h"
#include "mlir/ral/ral_context.h"
#include "mlir/ral/ral_helper.h"
#include "mlir/ral/ral_logging.h"

namespace tao {
namespace ral {
namespace gpu {
namespace io {

namespace {

BaseHipExecutionContext* execOf(ExecutionContext* ctx) {
  auto* exec = dynamic_cast<BaseHipExecutionContext*>(ctx);
  if (!exec) ctx->signalError(Context::FAILURE, "not a program execution context");
  return exec;
}

// "<anything>_<elem type, e.g. f32 / i8>_<d0xd1x...>": shape and element width of a
// constant are part of its name
bool parseConstName(const std::string& name, buffer_shape_t* shape, int64_t* width_in_bytes) {
  const size_t a = name.find('_');
  const size_t b = a == std::string::npos ? a : name.find('_', a + 1);
  if (b == std::string::npos || name.find('_', b + 1) != std::string::npos) return false;
  const std::string ty = name.substr(a + 1, b - a - 1);
  size_t digits = 0;
  while (digits < ty.size() && (ty[digits] < '0' || ty[digits] > '9')) ++digits;
  if (digits == ty.size()) return false;
  int64_t bits = 0;
  for (size_t i = digits; i < ty.size(); ++i) {
    if (ty[i] < '0' || ty[i] > '9') return false;
    bits = bits * 10 + (ty[i] - '0');
  }
  *width_in_bytes = bits / 8 < 1 ? 1 : bits / 8;
  shape->clear();
  const std::string dims = name.substr(b + 1);
  size_t pos = 0;
  while (pos < dims.size()) {
    size_t x = dims.find('x', pos);
    if (x == std::string::npos) x = dims.size();
    if (x == pos) return false;
    int64_t d = 0;
    for (size_t i = pos; i < x; ++i) {
      if (dims[i] < '0' || dims[i] > '9') return false;
      d = d * 10 + (dims[i] - '0');
    }
    shape->push_back(d);
    pos = x + 1;
  }
  return true;
}

int hexDigit(char c) {
  if (c >= '0' && c <= '9') return c - '0';
  if (c >= 'a' && c <= 'f') return c - 'a' + 10;
  if (c >= 'A' && c <= 'F') return c - 'A' + 10;
  return -1;
}

// hexadecimal text -> bytes; an odd-length string has an implied leading zero
bool fromHex(const std::string& text, std::vector<uint8_t>* out) {
  out->clear();
  out->reserve(text.size() / 2 + 1);
  size_t i = 0;
  if (text.size() % 2 == 1) {
    const int lo = hexDigit(text[0]);
    if (lo < 0) return false;
    out->push_back((uint8_t)lo);
    i = 1;
  }
  for (; i < text.size(); i += 2) {   // an even number of characters is left
    const int hi = hexDigit(text[i]), lo = hexDigit(text[i + 1]);
    if (hi < 0 || lo < 0) return false;
    out->push_back((uint8_t)((hi << 4) | lo));
  }
  return true;
}

// Bytes of constant `name`: decoded from the metadata file, a splat value repeated to
// the full size.
bool constantBytes(ExecutionContext* ctx, RalGlobalConstantState* state, const std::string& name,
                   bool host, buffer_shape_t* shape, std::vector<uint8_t>* bytes) {
  int64_t width = 0;
  if (!parseConstName(name, shape, &width)) {
    ctx->signalError(Context::FAILURE, "unexpected const unique_name format: " + name);
    return false;
  }
  const std::string* hex = nullptr;
  if (!state->metadata || !(host ? state->metadata->getHostConstant(name, hex)
                                 : state->metadata->getDeviceConstant(name, hex))) {
    ctx->signalError(Context::FAILURE, "const unique_name " + name + " not found in metadata file");
    return false;
  }
  if (!fromHex(*hex, bytes)) {
    ctx->signalError(Context::FAILURE, "const " + name + " is not a hexadecimal string");
    return false;
  }
  int64_t elems = 1;
  for (int64_t d : *shape) elems *= d;
  const size_t want = (size_t)(elems * width);
  if (bytes->size() < want && !bytes->empty()) {   // splat
    const std::vector<uint8_t> unit = *bytes;
    bytes->reserve(want);
    while (bytes->size() < want) bytes->insert(bytes->end(), unit.begin(), unit.end());
    bytes->resize(want);
  }
  return true;
}

buffer_t deviceConstant(ExecutionContext* ctx, void* stream_handle, const char* unique_name,
                        buffer_shape_t** shape) {
  auto* state = ctx->getResource<RalGlobalConstantState>(kRalGlobalConstantState);
  if (!state || !unique_name) {
    ctx->signalError(Context::FAILURE, "ral_const: no constant store");
    return nullptr;
  }
  // the process-level store, if enabled, in place of the context's own
  // (R context/common_context_impl_cuda.cc:66-73, 119-121)
  const bool shared = state->process_level_store != nullptr;
  if (shared) state = &state->process_level_store->state;
  std::lock_guard<std::mutex> guard(state->mu);
  const std::string key(unique_name);
  auto it = state->device_constants.find(key);
  if (it == state->device_constants.end()) {
    buffer_shape_t dims;
    std::vector<uint8_t> bytes;
    if (!constantBytes(ctx, state, key, false, &dims, &bytes)) return nullptr;
    auto* drv = ctx->getDriver<GPUDriver>(GPUDriver::name());
    const size_t size = bytes.empty() ? 1 : bytes.size();
    buffer_t dev = shared ? processLevelDeviceAlloc(size) : drv->alloc_persistent(ctx, size);
    if (!dev) return nullptr;
    if (!bytes.empty()) {
      drv->h2d(ctx, stream_handle, bytes.data(), dev, bytes.size());
      drv->syncOnStream(ctx, stream_handle);   // `bytes` dies with this scope
    }
    state->metadata->releaseDeviceConstant(key);
    it = state->device_constants.emplace(key, std::make_pair(dev, dims)).first;
    state->device_constant_buffers.insert(dev);
  }
  *shape = &it->second.second;
  return it->second.first;
}

buffer_t hostConstant(ExecutionContext* ctx, const char* unique_name, buffer_shape_t** shape) {
  auto* state = ctx->getResource<RalGlobalConstantState>(kRalGlobalConstantState);
  if (!state || !unique_name) {
    ctx->signalError(Context::FAILURE, "ral_const: no constant store");
    return nullptr;
  }
  if (state->process_level_store) state = &state->process_level_store->state;
  std::lock_guard<std::mutex> guard(state->mu);
  const std::string key(unique_name);
  auto it = state->host_constants.find(key);
  if (it == state->host_constants.end()) {
    buffer_shape_t dims;
    std::vector<uint8_t> bytes;
    if (!constantBytes(ctx, state, key, true, &dims, &bytes)) return nullptr;
    void* mem = ::operator new(bytes.empty() ? 1 : bytes.size());
    if (!bytes.empty()) std::memcpy(mem, bytes.data(), bytes.size());
    state->metadata->releaseHostConstant(key);
    it = state->host_constants.emplace(key, std::make_pair(mem, dims)).first;
  }
  *shape = &it->second.second;
  return it->second.first;
}

}  // namespace

// ------------------------------------------------------------ inputs / outputs
template <typename T, int N>
MemRefType<T, N> ral_recv_input(ExecutionContext* ctx, int64_t input_idx) {
  int64_t zeros[N > 0 ? N : 1] = {0};
  MemRefType<T, N> none = assignMemRef<T, N>(nullptr, zeros);
  auto* exec = execOf(ctx);
  if (!exec) return none;
  auto it = exec->inputs.find((int32_t)input_idx);
  if (it == exec->inputs.end() || (int)it->second.shape.size() != N) {
    ctx->signalError(Context::FAILURE, it == exec->inputs.end() ? "invalid input index"
                                                                  : "input rank mismatch");
    return none;
  }
  return assignMemRef<T, N>(it->second.buffer, it->second.shape);
}

template <typename T>
MemRefType<T, 0> ral_recv_input_0d(ExecutionContext* ctx, int64_t input_idx) {
  MemRefType<T, 0> none = assignMemRef_0d<T>(nullptr);
  auto* exec = execOf(ctx);
  if (!exec) return none;
  auto it = exec->inputs.find((int32_t)input_idx);
  if (it == exec->inputs.end()) {
    ctx->signalError(Context::FAILURE, "invalid input index");
    return none;
  }
  return assignMemRef_0d<T>(it->second.buffer);
}

template <typename T, int N>
void ral_send_output(ExecutionContext* ctx, int64_t output_idx, MemRefType<T, N> memref) {
  auto* exec = execOf(ctx);
  if (!exec) return;
  Tensor t;
  t.buffer = memref.data;
  for (int i = 0; i < N; ++i) t.shape.push_back(memref.sizes[i]);
  if (exec->outputs.emplace((int32_t)output_idx, std::move(t)).second)
    ++exec->outputSharedOrder[memref.data];
}

template <typename T>
void ral_send_output_0d(ExecutionContext* ctx, int64_t output_idx, MemRefType<T, 0> memref) {
  auto* exec = execOf(ctx);
  if (!exec) return;
  Tensor t;
  t.buffer = memref.data;
  if (exec->outputs.emplace((int32_t)output_idx, std::move(t)).second)
    ++exec->outputSharedOrder[memref.data];
}

// ------------------------------------------------------------------- constants
template <typename T, int N>
MemRefType<T, N> ral_const_device(ExecutionContext* ctx, void* stream_handle,
                                  const char* unique_name, int32_t /*unique_index_in_module*/) {
  int64_t zeros[N > 0 ? N : 1] = {0};
  buffer_shape_t* shape = nullptr;
  buffer_t ptr = deviceConstant(ctx, stream_handle, unique_name, &shape);
  if (!ptr || !shape || (int)shape->size() != N) {
    if (ptr) ctx->signalError(Context::FAILURE, "unexpected shape string in unique_name");
    return assignMemRef<T, N>(nullptr, zeros);
  }
  return assignMemRef<T, N>(ptr, *shape);
}

template <typename T>
MemRefType<T, 0> ral_const_device_0d(ExecutionContext* ctx, void* stream_handle,
                                     const char* unique_name, int32_t) {
  buffer_shape_t* shape = nullptr;
  buffer_t ptr = deviceConstant(ctx, stream_handle, unique_name, &shape);
  if (!ptr || !shape || !shape->empty()) {
    if (ptr) ctx->signalError(Context::FAILURE, "unexpected shape string in unique_name");
    return assignMemRef_0d<T>(nullptr);
  }
  return assignMemRef_0d<T>(ptr);
}

template <typename T, int N>
MemRefType<T, N> ral_const_host(ExecutionContext* ctx, void* /*stream_handle*/,
                                const char* unique_name, int32_t) {
  int64_t zeros[N > 0 ? N : 1] = {0};
  buffer_shape_t* shape = nullptr;
  buffer_t ptr = hostConstant(ctx, unique_name, &shape);
  if (!ptr || !shape || (int)shape->size() != N) {
    if (ptr) ctx->signalError(Context::FAILURE, "unexpected shape string in unique_name");
    return assignMemRef<T, N>(nullptr, zeros);
  }
  return assignMemRef<T, N>(ptr, *shape);
}

template <typename T>
MemRefType<T, 0> ral_const_host_0d(ExecutionContext* ctx, void*, const char* unique_name,
                                   int32_t) {
  buffer_shape_t* shape = nullptr;
  buffer_t ptr = hostConstant(ctx, unique_name, &shape);
  if (!ptr || !shape || !shape->empty()) {
    if (ptr) ctx->signalError(Context::FAILURE, "unexpected shape string in unique_name");
    return assignMemRef_0d<T>(nullptr);
  }
  return assignMemRef_0d<T>(ptr);
}

// --------------------------------------------------- inc_ref (reshape / alias)
// A second memref over the same buffer: one more reference on a buffer of this
// execution; inputs and persistent buffers are pinned so that a later dealloc of the
// alias never frees them.
namespace {
void addReference(ExecutionContext* ctx, buffer_t ptr) {
  auto* exec = execOf(ctx);
  if (!exec || !ptr) return;
  auto it = exec->device_ptr_map.find(ptr);
  if (it != exec->device_ptr_map.end()) {
    ++it->second;
  } else if (exec->input_ptr_set.count(ptr) || isPersistentDeviceBuffer(ctx, ptr)) {
    exec->device_ptr_map[ptr] = 2;
  } else {
    ctx->signalError(Context::FAILURE, "inc_ref: buffer is not known to this execution");
  }
}

// the same for host buffers (inc_ref on the cpu device, R context/base/cpu/
// cpu_context_impl.cc:232-255)
void addHostReference(ExecutionContext* ctx, buffer_t ptr) {
  auto* exec = execOf(ctx);
  if (!exec || !ptr) return;
  auto it = exec->host_ptr_map.find(ptr);
  if (it != exec->host_ptr_map.end()) {
    ++it->second;
    return;
  }
  bool persistent = false;
  if (auto* host = ctx->getResource<BaseHostContextState>(kRalBaseCpuContextState)) {
    std::lock_guard<std::mutex> guard(host->mu);
    persistent = host->host_persistent_buffers.count(ptr) != 0;
  }
  if (exec->input_ptr_set.count(ptr) || persistent) {
    exec->host_ptr_map[ptr] = 2;    // borrowed: never released through this alias
  } else {
    ctx->signalError(Context::FAILURE, "inc_ref: host buffer is not known to this execution");
  }
}
}  // namespace

template <typename T, int N>
MemRefType<T, N> ral_inc_ref_host(ExecutionContext* ctx, void*, MemRefType<T, N> input) {
  addHostReference(ctx, input.data);
  return input;
}

template <typename T, int N>
MemRefType<T, N> ral_inc_ref(ExecutionContext* ctx, void*, MemRefType<T, N> input) {
  addReference(ctx, input.data);
  return input;
}

template <typename T, int N, int M, bool HOST = false, typename P = int64_t>
MemRefType<T, M> ral_inc_ref_reshape(ExecutionContext* ctx, void*, MemRefType<T, N> input,
                                     MemRefType<P, 1> shape) {
  MemRefType<T, M> out;
  out.basePtr = input.basePtr;
  out.data = input.data;
  out.offset = 0;
  if (shape.sizes[0] != M) {
    ctx->signalError(Context::FAILURE, "inc_ref: shape operand has the wrong length");
    for (int i = 0; i < M; ++i) out.sizes[i] = out.strides[i] = 0;
    return out;
  }
  for (int i = 0; i < M; ++i) out.sizes[i] = (int64_t)shape.data[i];
  int64_t stride = 1;
  for (int i = M - 1; i >= 0; --i) {
    out.strides[i] = stride;
    stride *= out.sizes[i];
  }
  if (HOST)
    addHostReference(ctx, input.data);
  else
    addReference(ctx, input.data);
  return out;
}

// ------------------------------------------------------ memref-typed copies
template <typename T, int N>
int64_t byteSize(const MemRefType<T, N>& m) {
  int64_t n = 1;
  for (int i = 0; i < N; ++i) n *= m.sizes[i];
  return n * (int64_t)sizeof(T);
}

template <typename T, int N>
void ral_h2d_memref(ExecutionContext* ctx, void* stream_handle, MemRefType<T, N> from,
                    MemRefType<T, N> to) {
  const int64_t bytes = byteSize(from);
  if (bytes == 0) return;
  ctx->getDriver<GPUDriver>(GPUDriver::name())->h2d(ctx, stream_handle, from.data, to.data,
                                                   (size_t)bytes);
}

template <typename T, int N>
void ral_d2h_memref(ExecutionContext* ctx, void* stream_handle, MemRefType<T, N> from,
                    MemRefType<T, N> to) {
  const int64_t bytes = byteSize(from);
  if (bytes == 0) return;
  ctx->getDriver<GPUDriver>(GPUDriver::name())->d2h(ctx, stream_handle, from.data, to.data,
                                                   (size_t)bytes);
}

template <typename T, int N>
void ral_d2d_memref(ExecutionContext* ctx, void* stream_handle, MemRefType<T, N> from,
                    MemRefType<T, N> to) {
  const int64_t bytes = byteSize(from);
  if (bytes == 0) return;
  ctx->getDriver<GPUDriver>(GPUDriver::name())->d2d(ctx, stream_handle, from.data, to.data,
                                                   (size_t)bytes);
}

}  // namespace io
}  // namespace gpu

// -------------------------------------------------------------- registrations
#define RAL_IO_FOR_RANK(T, N)                                                        \
  TAO_RAL_API(tao::ral::kRalRecvInput, "cpu", gpu::io::ral_recv_input<T, N>);        \
  TAO_RAL_API(tao::ral::kRalSendOutput, "cpu", gpu::io::ral_send_output<T, N>);      \
  TAO_RAL_API(tao::ral::kRalCudaConst, "gpu", gpu::io::ral_const_device<T, N>);      \
  TAO_RAL_API(tao::ral::kRalHostConst, "cpu", gpu::io::ral_const_host<T, N>);        \
  TAO_RAL_API(tao::ral::kRalBitcast, "gpu", gpu::io::ral_inc_ref<T, N>);             \
  TAO_RAL_API(tao::ral::kRalBitcast, "cpu", gpu::io::ral_inc_ref_host<T, N>);        \
  TAO_RAL_API("h2d", "gpu", gpu::io::ral_h2d_memref<T, N>);                          \
  TAO_RAL_API("d2h", "gpu", gpu::io::ral_d2h_memref<T, N>);                          \
  TAO_RAL_API("d2d", "gpu", gpu::io::ral_d2d_memref<T, N>);

#define RAL_IO_RESHAPE(T, N, M)                                                      \
  TAO_RAL_API(tao::ral::kRalBitcast, "gpu", gpu::io::ral_inc_ref_reshape<T, N, M>); \
  TAO_RAL_API(tao::ral::kRalBitcast, "cpu", (gpu::io::ral_inc_ref_reshape<T, N, M, true>));

#define RAL_IO_FOR_TYPE(T)                                                           \
  TAO_RAL_API(tao::ral::kRalRecvInput, "cpu", gpu::io::ral_recv_input_0d<T>);        \
  TAO_RAL_API(tao::ral::kRalSendOutput, "cpu", gpu::io::ral_send_output_0d<T>);      \
  TAO_RAL_API(tao::ral::kRalCudaConst, "gpu", gpu::io::ral_const_device_0d<T>);      \
  TAO_RAL_API(tao::ral::kRalHostConst, "cpu", gpu::io::ral_const_host_0d<T>);        \
  RAL_IO_FOR_RANK(T, 1) RAL_IO_FOR_RANK(T, 2) RAL_IO_FOR_RANK(T, 3) RAL_IO_FOR_RANK(T, 4) \
  RAL_IO_RESHAPE(T, 1, 2) RAL_IO_RESHAPE(T, 1, 3) RAL_IO_RESHAPE(T, 1, 4)            \
  RAL_IO_RESHAPE(T, 2, 1) RAL_IO_RESHAPE(T, 2, 3) RAL_IO_RESHAPE(T, 2, 4)            \
  RAL_IO_RESHAPE(T, 3, 1) RAL_IO_RESHAPE(T, 3, 2) RAL_IO_RESHAPE(T, 3, 4)            \
  RAL_IO_RESHAPE(T, 4, 1) RAL_IO_RESHAPE(T, 4, 2) RAL_IO_RESHAPE(T, 4, 3)

// the element types a quantized inference program moves around
RAL_IO_FOR_TYPE(float);
RAL_IO_FOR_TYPE(int8_t);
RAL_IO_FOR_TYPE(uint8_t);
RAL_IO_FOR_TYPE(int32_t);
RAL_IO_FOR_TYPE(int64_t);
RAL_IO_FOR_TYPE(bool);

}  // namespace ral
}  // namespace tao
