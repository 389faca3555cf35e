// C entry points of the runtime plugin ABI (include/tao_ral_api.h).
#include "tao_ral_api.h"

#include <mutex>
#include <string>
#include <vector>

#include <algorithm>
#include <cstring>
#include <sstream>

#include "mlir/ral/context/base/hip/hip_context_impl.h"
#include "mlir/ral/context/conv_attr_util.h"
#include "mlir/ral/context/pdll_util.h"
#include "mlir/ral/ral_context.h"
#include "mlir/ral/ral_helper.h"
#include "mlir/ral/ral_logging.h"
#include "mlir/ral/ral_metadata.h"

namespace {

// Allocator over a pair of C callbacks supplied by the embedding framework.
class CallbackAllocator : public tao::ral::Allocator {
 public:
  CallbackAllocator(disc_ral_alloc_fn a, disc_ral_dealloc_fn d, void* user)
      : alloc_(a), dealloc_(d), user_(user) {}
  tao::ral::buffer_t alloc(size_t bytes) override { return alloc_(bytes, user_); }
  void dealloc(tao::ral::buffer_t p) override { dealloc_(p, user_); }

 private:
  disc_ral_alloc_fn alloc_;
  disc_ral_dealloc_fn dealloc_;
  void* user_;
};

std::vector<std::string>& apiNames() {
  static std::vector<std::string> names;
  static std::once_flag once;
  std::call_once(once, [] { names = tao::ral::TaoRalApiRegistry::Global().Names(); });
  return names;
}

void renderJson(tao::ral::PDLAttr& a, std::ostringstream& os) {
  using namespace tao::ral;
  const std::string& t = a.getType();
  auto quote = [&](const std::string& s) {
    os << '"';
    for (char c : s) {
      if (c == '"' || c == '\\') os << '\\';
      os << c;
    }
    os << '"';
  };
  if (t == "dict") {
    auto& items = a.as<DictPDLAttr>().getValue();
    std::vector<std::string> keys;
    for (auto& kv : items) keys.push_back(kv.first);
    std::sort(keys.begin(), keys.end());
    os << '{';
    for (size_t i = 0; i < keys.size(); ++i) {
      if (i) os << ", ";
      quote(keys[i]);
      os << ": ";
      renderJson(*items[keys[i]], os);
    }
    os << '}';
  } else if (t == "str") {
    quote(a.as<StrPDLAttr>().getValue());
  } else if (t == "bool") {
    os << (a.as<BoolPDLAttr>().getValue() ? "true" : "false");
  } else if (t == "int") {
    os << a.as<IntPDLAttr>().getValue();
  } else if (t == "float") {
    os.precision(17);
    os << a.as<FloatPDLAttr>().getValue();
  } else if (t == "intArray") {
    auto& v = a.as<IntArrayPDLAttr>().getValue();
    os << '[';
    for (size_t i = 0; i < v.size(); ++i) os << (i ? ", " : "") << v[i];
    os << ']';
  } else if (t == "array") {
    auto& v = a.as<ArrayPDLAttr>().getValue();
    os << '[';
    for (size_t i = 0; i < v.size(); ++i) {
      if (i) os << ", ";
      renderJson(*v[i], os);
    }
    os << ']';
  } else if (t == "denseElementsAttr") {
    auto& d = a.as<DenseElementsPDLAttr>();
    os << "{\"dense\": ";
    quote(d.getElementType() + std::to_string(d.getNumBits()));
    os << ", \"shape\": [";
    auto shape = d.getShape();
    for (size_t i = 0; i < shape.size(); ++i) os << (i ? ", " : "") << shape[i];
    os << "], \"bytes\": [";
    auto& raw = d.getRawData();
    for (size_t i = 0; i < raw.size(); ++i) os << (i ? ", " : "") << (int)raw[i];
    os << "]}";
  }
}

}  // namespace

extern "C" {

const char* const kMlirLoweredEntry = "main";

void tao_ral_call_impl(tao_ral_context_t ctx, void* name, void** args) {
  auto* exec = static_cast<tao::ral::ExecutionContext*>(ctx);
  TAO_VLOG(1) << "tao_ral_call: " << static_cast<const char*>(name);
  exec->getContext()->call(static_cast<const char*>(name), args);
}

tao_ral_status_t tao_ral_last_error(tao_ral_context_t ctx, const char** err_msg) {
  return static_cast<tao::ral::Context*>(ctx)->getLastError(err_msg);
}

void tao_ral_clear_error(tao_ral_context_t ctx) {
  static_cast<tao::ral::Context*>(ctx)->clearError();
}

tao_ral_context_t disc_ral_context_create(void* hip_stream, int device_ordinal,
                                          disc_ral_alloc_fn alloc,
                                          disc_ral_dealloc_fn dealloc, void* user,
                                          int cache_workspace) {
  return disc_ral_context_create_for_program(hip_stream, device_ordinal, alloc, dealloc, user,
                                             cache_workspace, nullptr);
}

tao_ral_context_t disc_ral_context_create_for_program(void* hip_stream, int device_ordinal,
                                                      disc_ral_alloc_fn alloc,
                                                      disc_ral_dealloc_fn dealloc, void* user,
                                                      int cache_workspace,
                                                      const char* metadata_file_path) {
  if ((alloc == nullptr) != (dealloc == nullptr)) return nullptr;
  tao::ral::BaseContextOption opt;
  if (metadata_file_path) opt.metadata_file_path = metadata_file_path;
  opt.cache_workspace_mem_across_execution = cache_workspace != 0;
  tao::ral::gpu::BaseHipContextOption gpu_opt;
  gpu_opt.stream = static_cast<hipStream_t>(hip_stream);
  gpu_opt.device_ordinal = device_ordinal;
  if (alloc) gpu_opt.gpu_allocator.reset(new CallbackAllocator(alloc, dealloc, user));
  auto ctx = tao::ral::gpu::MakeBaseHipContext(opt, gpu_opt);
  return static_cast<tao::ral::Context*>(ctx.release());
}

void disc_ral_context_destroy(tao_ral_context_t ctx) {
  delete static_cast<tao::ral::Context*>(ctx);
}

tao_ral_context_t disc_ral_execution_context_create(tao_ral_context_t ctx) {
  auto* base = dynamic_cast<tao::ral::BaseContext*>(static_cast<tao::ral::Context*>(ctx));
  if (!base) return nullptr;
  return static_cast<tao::ral::ExecutionContext*>(
      new tao::ral::gpu::BaseHipExecutionContext(base));
}

void disc_ral_execution_context_destroy(tao_ral_context_t exec_ctx) {
  delete static_cast<tao::ral::ExecutionContext*>(exec_ctx);
}

tao_ral_context_t disc_ral_execution_context_get_context(tao_ral_context_t exec_ctx) {
  return static_cast<tao::ral::ExecutionContext*>(exec_ctx)->getContext();
}

int disc_ral_execution_bind_input(tao_ral_context_t exec_ctx, int input_idx, void* buffer,
                                  const int64_t* shape, int rank) {
  auto* exec = static_cast<tao::ral::ExecutionContext*>(exec_ctx);
  if (!exec || rank < 0 || (rank > 0 && !shape)) return 1;
  exec->bindInput(input_idx, buffer, tao::ral::buffer_shape_t(shape, shape + rank));
  return 0;
}

disc_ral_output_t disc_ral_execution_take_output(tao_ral_context_t exec_ctx, int output_idx) {
  auto* exec = static_cast<tao::ral::ExecutionContext*>(exec_ctx);
  if (!exec) return nullptr;
  std::unique_ptr<tao::ral::OutputBufferWrapper> out;
  exec->bindOutput(output_idx, &out);
  return out.release();
}

const void* disc_ral_output_data(disc_ral_output_t output) {
  return output ? static_cast<tao::ral::OutputBufferWrapper*>(output)->data() : nullptr;
}

int disc_ral_output_rank(disc_ral_output_t output) {
  return output ? (int)static_cast<tao::ral::OutputBufferWrapper*>(output)->shape().size() : -1;
}

int64_t disc_ral_output_dim(disc_ral_output_t output, int i) {
  if (!output) return -1;
  const auto& shape = static_cast<tao::ral::OutputBufferWrapper*>(output)->shape();
  return i >= 0 && i < (int)shape.size() ? shape[i] : -1;
}

int disc_ral_output_owned(disc_ral_output_t output) {
  return output && static_cast<tao::ral::OutputBufferWrapper*>(output)->owned() ? 1 : 0;
}

void disc_ral_output_release(disc_ral_output_t output) {
  if (output) static_cast<tao::ral::OutputBufferWrapper*>(output)->release();
}

void disc_ral_output_destroy(disc_ral_output_t output) {
  delete static_cast<tao::ral::OutputBufferWrapper*>(output);
}

int disc_ral_metadata_emit(const char* path, int count, const uint8_t* is_host,
                           const char* const* names, const char* const* hex_values) {
  if (!path || count < 0 || (count > 0 && (!is_host || !names || !hex_values))) return 1;
  tao::ral::MetadataFileEmitter emitter(path);
  if (!emitter.emitHeader()) return 1;
  for (int i = 0; i < count; ++i) {
    if (!names[i] || !hex_values[i]) return 1;
    const bool ok = is_host[i] ? emitter.emitHostConstant(names[i], hex_values[i])
                               : emitter.emitDeviceConstant(names[i], hex_values[i]);
    if (!ok) return 1;
  }
  return emitter.emitTailer() ? 0 : 1;
}

int disc_ral_metadata_count(const char* path, int* host_constants, int* device_constants,
                            const char* const* probe_names, int n_probe) {
  auto file = path ? tao::ral::MetadataFile::loadFromFile(path) : nullptr;
  if (!file) return 1;
  int h = 0, d = 0;
  for (int i = 0; i < n_probe; ++i) {
    const std::string* data = nullptr;
    if (probe_names[i] && file->getHostConstant(probe_names[i], data)) ++h;
    if (probe_names[i] && file->getDeviceConstant(probe_names[i], data)) ++d;
  }
  if (host_constants) *host_constants = h;
  if (device_constants) *device_constants = d;
  return 0;
}

int disc_ral_api_count(void) { return static_cast<int>(apiNames().size()); }

const char* disc_ral_api_name(int index) {
  auto& names = apiNames();
  if (index < 0 || index >= static_cast<int>(names.size())) return "";
  return names[index].c_str();
}

int disc_ral_api_exists(const char* name) {
  return name && tao::ral::TaoRalApiRegistry::Global().Find(name) ? 1 : 0;
}

int disc_ral_conv2d_plan(const char* data_format, const int64_t* strides, int n_strides,
                         const int64_t* dilations, int n_dilations, const char* padding,
                         const int64_t* explicit_paddings, int n_explicit,
                         int weight_is_const, const int64_t in_sizes[4],
                         const int64_t w_sizes[4], int32_t padding_out[4],
                         int32_t metadata_out[17], int64_t result_sizes_out[4]) {
  if (!data_format || !padding || !in_sizes || !w_sizes || !padding_out || !metadata_out ||
      !result_sizes_out || n_strides < 0 || n_dilations < 0 || n_explicit < 0)
    return 1;
  tao::ral::Conv2dPlan plan;
  const std::string err = tao::ral::planConv2d(
      data_format, std::vector<int64_t>(strides, strides + n_strides),
      std::vector<int64_t>(dilations, dilations + n_dilations), padding,
      std::vector<int64_t>(explicit_paddings, explicit_paddings + n_explicit),
      weight_is_const != 0, in_sizes, w_sizes, &plan);
  if (!err.empty()) return 1;
  std::memcpy(padding_out, plan.padding, sizeof(plan.padding));
  std::memcpy(metadata_out, plan.metadata, sizeof(plan.metadata));
  std::memcpy(result_sizes_out, plan.result_sizes, sizeof(plan.result_sizes));
  return 0;
}

int64_t disc_ral_attr_to_json(const uint8_t* blob, size_t size, char* out, size_t cap) {
  if (!blob) return -1;
  size_t used = 0;
  auto attr = tao::ral::parsePDLAttr(blob, size, &used);
  if (!attr) return -1;
  std::ostringstream os;
  renderJson(*attr, os);
  const std::string text = os.str();
  if (out && cap) {
    const size_t n = std::min(cap - 1, text.size());
    std::memcpy(out, text.data(), n);
    out[n] = 0;
  }
  return static_cast<int64_t>(text.size());
}

}  // extern "C"
