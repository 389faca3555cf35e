#include "mlir/ral/context/base/hip/hip_context_impl.h"

#include <cstring>
#include <cstdlib>
#include <cctype>
#include <algorithm>
#include <mutex>
#include <sstream>
#include <unordered_set>

#include "disc_q8.h"
#include "mlir/ral/ral_helper.h"
#include "mlir/ral/ral_logging.h"

namespace tao {
namespace ral {

BaseContext::BaseContext(BaseContextOption& opt) : opt_(opt) {}
BaseContext::~BaseContext() = default;

// ------------------------------------------------------------ InternalAllocator
InternalAllocator::InternalAllocator(alloc_t alloc_func, dealloc_t dealloc_func)
    : alloc_func_(std::move(alloc_func)), dealloc_func_(std::move(dealloc_func)) {}

InternalAllocator::~InternalAllocator() {
  releaseAllFreeBuffers();
  // anything still live is returned too: the context is going away
  for (auto& kv : class_of_) dealloc_func_(kv.first);
}

size_t InternalAllocator::sizeClass(size_t bytes) {
  constexpr size_t kMin = 256;
  if (bytes <= kMin) return kMin;
  size_t pow2 = kMin;
  while (pow2 < bytes) pow2 <<= 1;        // smallest power of two >= bytes
  const size_t quarter = pow2 >> 3;       // steps of 1/4 of the lower power
  size_t cls = pow2 >> 1;
  while (cls < bytes) cls += quarter;
  return cls;
}

void InternalAllocator::releaseAllFreeBuffers() {
  for (auto& kv : free_by_class_)
    for (buffer_t b : kv.second) {
      dealloc_func_(b);
      class_of_.erase(b);
    }
  free_by_class_.clear();
  pooled_bytes_ = 0;
}

buffer_t InternalAllocator::alloc(size_t bytes) {
  const size_t cls = sizeClass(bytes);
  auto it = free_by_class_.find(cls);
  if (it != free_by_class_.end() && !it->second.empty()) {
    buffer_t b = it->second.back();
    it->second.pop_back();
    pooled_bytes_ -= cls;
    live_bytes_ += cls;
    return b;
  }
  buffer_t b = alloc_func_(cls);
  if (!b) {  // give the pool back to the device and retry once
    releaseAllFreeBuffers();
    b = alloc_func_(cls);
    if (!b) return nullptr;
  }
  class_of_[b] = cls;
  live_bytes_ += cls;
  return b;
}

void InternalAllocator::dealloc(buffer_t buffer) {
  auto it = class_of_.find(buffer);
  if (it == class_of_.end()) return;  // not ours
  free_by_class_[it->second].push_back(buffer);
  live_bytes_ -= it->second;
  pooled_bytes_ += it->second;
}

namespace gpu {

const char* kRalBaseHipContextState = "ral_base_hip_context_state";
const char* kRalGlobalConstantState = "ral_global_constant_state";

namespace {

bool hipOk(hipError_t e, ExecutionContext* ctx, const char* where) {
  if (e == hipSuccess) return true;
  // The error is reported through the context; take it off the thread's HIP error state so
  // that the framework sharing this thread does not trip over it at its next GPU call.
  (void)hipGetLastError();
  std::ostringstream out;
  out << "GPU failed with " << hipGetErrorString(e) << " in " << where;
  ctx->signalError(Context::FAILURE, out.str());
  return false;
}

struct BaseHipContextState : public Context::Resource {
  std::mutex mu;
  GpuStreamHandle stream = nullptr;
  int device_ordinal = 0;
  std::shared_ptr<Allocator> gpu_allocator;
  bool cache_workspace_mem_across_execution = false;
  std::unordered_set<const_buffer_t> device_persistent_buffers;
  // code objects of compiler-generated kernels: blob -> module, (blob,name) -> fn
  std::map<void*, hipModule_t> modules;
  std::map<std::pair<void*, std::string>, hipFunction_t> functions;

  void onExecutionFinish(ExecutionContext*) override {
    std::lock_guard<std::mutex> guard(mu);
    if (!cache_workspace_mem_across_execution) gpu_allocator->releaseAllFreeBuffers();
  }

  void onContextFinish(Context*) override {
    (void)hipStreamSynchronize(stream);
    for (const_buffer_t b : device_persistent_buffers)
      gpu_allocator->dealloc(const_cast<buffer_t>(b));
    device_persistent_buffers.clear();
    for (auto& kv : modules) (void)hipModuleUnload(kv.second);
    modules.clear();
    functions.clear();
    gpu_allocator->releaseAllFreeBuffers();
  }
};

BaseHipContextState* stateOf(ExecutionContext* ctx) {
  return ctx->getResource<BaseHipContextState>(kRalBaseHipContextState);
}

bool validStream(ExecutionContext* ctx, stream_t sidx) {
  if (reinterpret_cast<intptr_t>(sidx) == 0) return true;
  ctx->signalError(Context::FAILURE, "not a valid stream idx");
  return false;
}

// ---------------------------------------------------------- driver functions
buffer_t ral_base_hip_alloc(ExecutionContext* ctx, size_t bytes) {
  auto* state = stateOf(ctx);
  if (!state) return nullptr;
  auto* exec = dynamic_cast<BaseHipExecutionContext*>(ctx);
  if (!exec) {
    ctx->signalError(Context::FAILURE, "alloc needs a BaseHipExecutionContext");
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(state->mu);
  void* ptr = state->gpu_allocator->alloc(bytes ? bytes : 1);
  if (!ptr) {
    ctx->signalError(Context::FAILURE, "device allocation of " + std::to_string(bytes) +
                                           " bytes failed");
    return nullptr;
  }
  exec->device_ptr_map[ptr] = 1;
  return ptr;
}

buffer_t ral_base_hip_alloc_persistent(ExecutionContext* ctx, size_t bytes) {
  auto* state = stateOf(ctx);
  if (!state) return nullptr;
  std::lock_guard<std::mutex> guard(state->mu);
  void* ptr = state->gpu_allocator->alloc(bytes ? bytes : 1);
  if (!ptr) {
    ctx->signalError(Context::FAILURE, "persistent device allocation of " +
                                           std::to_string(bytes) + " bytes failed");
    return nullptr;
  }
  state->device_persistent_buffers.insert(ptr);
  return ptr;
}

void ral_base_hip_dealloc(ExecutionContext* ctx, buffer_t buffer) {
  if (!buffer) return;
  auto* state = stateOf(ctx);
  if (!state) return;
  auto* exec = dynamic_cast<BaseHipExecutionContext*>(ctx);
  std::lock_guard<std::mutex> guard(state->mu);
  if (state->device_persistent_buffers.count(buffer)) return;
  if (!exec) return;
  auto it = exec->device_ptr_map.find(buffer);
  if (it == exec->device_ptr_map.end()) {
    TAO_VLOG(1) << "dealloc: ignoring a buffer this execution did not allocate";
    return;
  }
  if (--it->second == 0) {
    // an alias of a program input was pinned by inc_ref; the buffer is the caller's
    if (!exec->input_ptr_set.count(buffer)) state->gpu_allocator->dealloc(buffer);
    exec->device_ptr_map.erase(it);
  }
}

buffer_t ral_base_hip_raw_alloc(Context* ctx, size_t bytes) {
  auto* state = static_cast<BaseHipContextState*>(
      ctx->getOrCreateResource(kRalBaseHipContextState, nullptr).get());
  if (!state) return nullptr;
  std::lock_guard<std::mutex> guard(state->mu);
  return state->gpu_allocator->alloc(bytes ? bytes : 1);
}

void ral_base_hip_raw_dealloc(Context* ctx, buffer_t buffer) {
  if (!buffer) return;
  auto* state = static_cast<BaseHipContextState*>(
      ctx->getOrCreateResource(kRalBaseHipContextState, nullptr).get());
  if (!state) return;
  std::lock_guard<std::mutex> guard(state->mu);
  state->gpu_allocator->dealloc(buffer);
}

namespace {
// True if the image at `blob` carries device code for gfx950: an AMDGPU ELF whose e_flags name
// that processor, or a clang offload bundle with an entry whose target ends in it.  Only the
// headers are read (a launch receives its images without their sizes).
bool codeObjectIsForGfx950(const void* blob) {
  const unsigned char* b = static_cast<const unsigned char*>(blob);
  auto u16 = [&](size_t o) { return (uint32_t)b[o] | ((uint32_t)b[o + 1] << 8); };
  auto u64 = [&](size_t o) {
    uint64_t v = 0;
    for (int i = 7; i >= 0; --i) v = (v << 8) | b[o + i];
    return v;
  };
  if (b[0] == 0x7f && b[1] == 'E' && b[2] == 'L' && b[3] == 'F') {
    constexpr uint32_t kEmAmdgpu = 224, kMachGfx950 = 0x4f;   // EF_AMDGPU_MACH: e_flags & 0xff
    return b[4] == 2 /* ELFCLASS64 */ && u16(18) == kEmAmdgpu && b[48] == kMachGfx950;
  }
  static const char kBundle[] = "__CLANG_OFFLOAD_BUNDLE__";
  if (std::memcmp(b, kBundle, 24) == 0) {
    // magic[24], u64 entries, then per entry u64 offset, u64 size, u64 triple length, triple
    const uint64_t entries = u64(24);
    size_t o = 32;
    for (uint64_t e = 0; e < entries && e < 64; ++e) {
      const uint64_t size = u64(o + 8), len = u64(o + 16);
      if (len > 256) return false;
      const std::string triple(reinterpret_cast<const char*>(b + o + 24), (size_t)len);
      o += 24 + (size_t)len;
      if (size == 0 || triple.compare(0, 4, "host") == 0) continue;
      // "hipv4-amdgcn-amd-amdhsa--gfx950" with optional ":feature" suffixes
      const size_t at = triple.rfind("gfx950");
      if (at != std::string::npos && at > 0 && triple[at - 1] == '-' &&
          (at + 6 == triple.size() || triple[at + 6] == ':'))
        return true;
    }
  }
  return false;
}
}  // namespace

void ral_base_hip_launch(ExecutionContext* ctx, void** blobs, size_t num_blobs,
                         const char* kernel_name, intptr_t gridX, intptr_t gridY,
                         intptr_t gridZ, intptr_t blockX, intptr_t blockY,
                         intptr_t blockZ, int32_t smem, void* stream_handle,
                         int32_t /*num_args*/, void** params) {
  if (!blockX || !blockY || !blockZ || !gridX || !gridY || !gridZ) return;  // empty
  auto* state = stateOf(ctx);
  if (!state || !validStream(ctx, stream_handle)) return;
  if (num_blobs < 1 || !blobs || !blobs[0]) {
    ctx->signalError(Context::FAILURE, "ral_kernel_launch: no code object");
    return;
  }
  // One blob is taken as it is; of several (the reference's builds for NVIDIA carry one image
  // per compute capability and pick by the device's, R context/base/cuda/
  // cuda_context_impl.cc:375-392) the first that holds gfx950 code.
  void* blob = blobs[0];
  if (num_blobs > 1) {
    blob = nullptr;
    for (size_t i = 0; i < num_blobs && !blob; ++i)
      if (blobs[i] && codeObjectIsForGfx950(blobs[i])) blob = blobs[i];
    if (!blob) {
      ctx->signalError(Context::FAILURE, "ral_kernel_launch: none of the " +
                                             std::to_string(num_blobs) +
                                             " code objects of kernel " + kernel_name +
                                             " is built for gfx950");
      return;
    }
  }
  hipFunction_t fn = nullptr;
  {
    std::lock_guard<std::mutex> guard(state->mu);
    auto key = std::make_pair(blob, std::string(kernel_name));
    auto fit = state->functions.find(key);
    if (fit == state->functions.end()) {
      auto mit = state->modules.find(blob);
      if (mit == state->modules.end()) {
        hipModule_t mod = nullptr;
        if (!hipOk(hipModuleLoadData(&mod, blob), ctx, "ModuleLoad")) return;
        mit = state->modules.emplace(blob, mod).first;
      }
      if (!hipOk(hipModuleGetFunction(&fn, mit->second, kernel_name), ctx, "GetFunction"))
        return;
      fit = state->functions.emplace(key, fn).first;
    }
    fn = fit->second;
  }
  hipOk(hipModuleLaunchKernel(fn, (unsigned)gridX, (unsigned)gridY, (unsigned)gridZ,
                              (unsigned)blockX, (unsigned)blockY, (unsigned)blockZ,
                              (unsigned)smem, state->stream, params, nullptr),
        ctx, "LaunchKernel");
}

stream_t ral_base_hip_get_stream(ExecutionContext* ctx, int32_t stream_id) {
  if (stream_id < 0) {
    ctx->signalError(Context::FAILURE, "not a valid stream_id");
    return nullptr;
  }
  if (stream_id > 0) {
    ctx->signalError(Context::FAILURE, "multi-stream not supported");
    return nullptr;
  }
  return reinterpret_cast<stream_t>(static_cast<intptr_t>(stream_id));
}

opaque_t ral_base_hip_as_cu_stream(ExecutionContext* ctx, stream_t) {
  auto* state = stateOf(ctx);
  return state ? state->stream : nullptr;
}

opaque_t ral_base_hip_as_se_stream(ExecutionContext*, stream_t) { return nullptr; }

void ral_base_hip_d2d(ExecutionContext* ctx, stream_t sidx, buffer_t from, buffer_t to,
                      size_t bytes) {
  auto* state = stateOf(ctx);
  if (!state || !validStream(ctx, sidx) || !bytes) return;
  hipOk(hipMemcpyAsync(to, from, bytes, hipMemcpyDeviceToDevice, state->stream), ctx, "d2d");
}

void ral_base_hip_d2h(ExecutionContext* ctx, stream_t sidx, buffer_t from, buffer_t to,
                      size_t bytes) {
  auto* state = stateOf(ctx);
  if (!state || !validStream(ctx, sidx) || !bytes) return;
  hipOk(hipMemcpyAsync(to, from, bytes, hipMemcpyDeviceToHost, state->stream), ctx, "d2h");
}

void ral_base_hip_h2d(ExecutionContext* ctx, stream_t sidx, const void* from, buffer_t to,
                      size_t bytes) {
  auto* state = stateOf(ctx);
  if (!state || !validStream(ctx, sidx) || !bytes) return;
  hipOk(hipMemcpyAsync(to, from, bytes, hipMemcpyHostToDevice, state->stream), ctx, "h2d");
}

void ral_base_hip_memset(ExecutionContext* ctx, stream_t sidx, buffer_t buffer, int value,
                         size_t bytes) {
  auto* state = stateOf(ctx);
  if (!state || !validStream(ctx, sidx) || !buffer || !bytes) return;
  // a fill kernel, not hipMemsetAsync: the launch may be recorded into a captured graph
  if (dq8_fill(buffer, value, bytes, state->stream) != 0)
    ctx->signalError(Context::FAILURE, std::string("GPU failed in memset: ") + dq8_last_error());
}

void ral_base_hip_sync_on_stream(ExecutionContext* ctx, stream_t sidx) {
  auto* state = stateOf(ctx);
  if (!state || !validStream(ctx, sidx)) return;
  hipOk(hipStreamSynchronize(state->stream), ctx, "StreamSync");
}

void ral_base_hip_sync_all(ExecutionContext* ctx) {
  hipOk(hipDeviceSynchronize(), ctx, "DeviceSync");
}

}  // namespace

BaseHipExecutionContext::BaseHipExecutionContext(BaseContext* ctx)
    : ExecutionContext(ctx) {
  onExecutionStart();
}

void BaseHipExecutionContext::bindInput(int input_idx, buffer_t buffer,
                                        const buffer_shape_t& shape) {
  Tensor t;
  t.buffer = buffer;
  t.shape = shape;
  inputs[input_idx] = std::move(t);
  input_ptr_set.insert(buffer);
}

void BaseHipExecutionContext::bindOutput(int output_idx,
                                         std::unique_ptr<OutputBufferWrapper>* output) {
  auto it = outputs.find(output_idx);
  if (it == outputs.end()) {
    signalError(Context::FAILURE, "output not found");
    return;
  }
  auto* wrapper = new BaseOutputBufferWrapper(it->second.buffer, it->second.shape);
  output->reset(wrapper);
  const_buffer_t buffer = it->second.buffer;
  // a buffer seen as an output before already has its deleter; a forwarded input or a
  // persistent buffer (a constant) is not the program's to free
  if (!output_ptr_set.insert(buffer).second) return;
  if (input_ptr_set.count(buffer)) return;
  auto* state = getResource<BaseHipContextState>(kRalBaseHipContextState);
  if (!state) return;
  std::lock_guard<std::mutex> guard(state->mu);
  if (state->device_persistent_buffers.count(buffer)) return;
  auto hit = host_ptr_map.find(buffer);
  if (hit != host_ptr_map.end()) {
    // a host output the program took from the cpu device's `alloc`
    if (--hit->second == 0) {
      wrapper->set_deleter([](buffer_t data) { std::free(data); });
      host_ptr_map.erase(hit);
    }
    if (outputSharedOrder[buffer] == 1) wrapper->markOwned();
    return;
  }
  auto dit = device_ptr_map.find(buffer);
  if (dit == device_ptr_map.end()) return;
  if (--dit->second == 0) {
    // the last reference leaves with the output: the wrapper returns it to the pool
    std::shared_ptr<Allocator> allocator = state->gpu_allocator;
    std::mutex* mu = &state->mu;
    wrapper->set_deleter([allocator, mu](buffer_t data) {
      std::lock_guard<std::mutex> g(*mu);
      allocator->dealloc(data);
    });
    device_ptr_map.erase(dit);
  }
  if (outputSharedOrder[buffer] == 1) wrapper->markOwned();
}

BaseHipExecutionContext::~BaseHipExecutionContext() {
  // Buffers the program allocated and never handed back return to the pool with the
  // execution.  The map also holds entries inc_ref pinned for aliases of program inputs and
  // of persistent buffers (constants, packed weights): those belong to the caller and to
  // the context and are left alone.
  auto* state = getResource<BaseHipContextState>(kRalBaseHipContextState);
  if (state) {
    std::lock_guard<std::mutex> guard(state->mu);
    for (auto& kv : device_ptr_map) {
      if (input_ptr_set.count(kv.first) || state->device_persistent_buffers.count(kv.first))
        continue;
      state->gpu_allocator->dealloc(const_cast<buffer_t>(kv.first));
    }
  }
  device_ptr_map.clear();
  auto* host = getResource<BaseHostContextState>(kRalBaseCpuContextState);
  for (auto& kv : host_ptr_map) {
    bool persistent = false;
    if (host) {
      std::lock_guard<std::mutex> guard(host->mu);
      persistent = host->host_persistent_buffers.count(kv.first) != 0;
    }
    if (!persistent && !input_ptr_set.count(kv.first)) std::free(const_cast<buffer_t>(kv.first));
  }
  host_ptr_map.clear();
  onExecutionFinish();
}

bool isPersistentDeviceBuffer(ExecutionContext* ctx, const_buffer_t buffer) {
  if (auto* state = ctx->getResource<BaseHipContextState>(kRalBaseHipContextState)) {
    std::lock_guard<std::mutex> guard(state->mu);
    if (state->device_persistent_buffers.count(buffer) != 0) return true;
  }
  // constants of the process-level store come from hipMalloc, not from this context
  if (auto* consts = ctx->getResource<RalGlobalConstantState>(kRalGlobalConstantState)) {
    if (ProcessLevelConstStore* store = consts->process_level_store) {
      std::lock_guard<std::mutex> guard(store->state.mu);
      return store->state.device_constant_buffers.count(buffer) != 0;
    }
  }
  return false;
}

buffer_t processLevelDeviceAlloc(size_t bytes) {
  void* p = nullptr;
  return hipMalloc(&p, bytes ? bytes : 1) == hipSuccess ? p : nullptr;
}

void processLevelDeviceFree(buffer_t buffer) {
  if (buffer) (void)hipFree(buffer);
}

bool discEnableGlobalConstantStore() {
  static const bool enabled = [] {
    const char* env = std::getenv("DISC_USE_GLOBAL_CONST_STORE");
    if (!env) return false;
    std::string v = env;
    std::transform(v.begin(), v.end(), v.begin(),
                   [](unsigned char c) { return (char)std::tolower(c); });
    return v == "true" || v == "1";
  }();
  return enabled;
}

ConstStoreRegistrar& ConstStoreRegistrar::Instance() {
  static ConstStoreRegistrar instance;
  return instance;
}

bool ConstStoreRegistrar::unregisterConstStore(ProcessLevelConstStore* store) {
  std::lock_guard<std::mutex> guard(mu);
  auto it = referenceCounter.find(store);
  if (it == referenceCounter.end()) return false;
  if (--it->second > 0) return false;
  pbFile2Instance.erase(store->pb_file_path);
  referenceCounter.erase(it);
  return true;
}

ProcessLevelConstStore* ConstStoreRegistrar::getConstStore(const std::string& pb_file_path) {
  std::lock_guard<std::mutex> guard(mu);
  auto it = pbFile2Instance.find(pb_file_path);
  if (it == pbFile2Instance.end()) {
    std::unique_ptr<ProcessLevelConstStore> store(new ProcessLevelConstStore);
    store->pb_file_path = pb_file_path;
    store->state.metadata = MetadataFile::loadFromFile(pb_file_path);
    if (!store->state.metadata) {
      TAO_LOG(ERROR) << "failed to load metadata file from: " << pb_file_path;
      return nullptr;
    }
    it = pbFile2Instance.emplace(pb_file_path, store.release()).first;
  }
  ++referenceCounter[it->second];
  return it->second;
}

void RalGlobalConstantState::onContextFinish(Context* ctx) {
  if (process_level_store) {
    // the last context to finish releases what the shared store holds
    ProcessLevelConstStore* store = process_level_store;
    process_level_store = nullptr;
    if (!ConstStoreRegistrar::Instance().unregisterConstStore(store)) return;
    (void)ctx;
    for (auto& kv : store->state.device_constants) processLevelDeviceFree(kv.second.first);
    for (auto& kv : store->state.host_constants) ::operator delete(kv.second.first);
    delete store;
    return;
  }
  // device constants come from alloc_persistent and go with the context state
  for (auto& kv : host_constants) ::operator delete(kv.second.first);
  host_constants.clear();
  device_constants.clear();
}

std::unique_ptr<BaseContext> MakeBaseHipContext(BaseContextOption& opt,
                                                BaseHipContextOption& gpu_opt) {
  std::unique_ptr<BaseContext> ctx(new BaseContext(opt));
  ctx->getOrCreateResource(kRalGlobalConstantState, [opt]() {
    auto* state = new RalGlobalConstantState;
    if (!opt.metadata_file_path.empty()) {
      if (discEnableGlobalConstantStore())
        state->process_level_store =
            ConstStoreRegistrar::Instance().getConstStore(opt.metadata_file_path);
      if (!state->process_level_store)
        state->metadata = MetadataFile::loadFromFile(opt.metadata_file_path);
    }
    return state;
  });
  ctx->addDriver(GPUDriver::name(), std::unique_ptr<GPUDriver>(new GPUDriver(ctx.get())));
  ctx->getOrCreateResource(kRalBaseCpuContextState, []() { return new BaseHostContextState; });
  ctx->getOrCreateResource(kRalBaseHipContextState, [opt, gpu_opt]() {
    auto* state = new BaseHipContextState;
    state->stream = gpu_opt.stream;
    state->device_ordinal = gpu_opt.device_ordinal;
    state->cache_workspace_mem_across_execution = opt.cache_workspace_mem_across_execution;
    if (gpu_opt.gpu_allocator) {
      state->gpu_allocator = gpu_opt.gpu_allocator;
    } else {
      state->gpu_allocator.reset(new InternalAllocator(
          [](size_t bytes) -> buffer_t {
            void* p = nullptr;
            return hipMalloc(&p, bytes) == hipSuccess ? p : nullptr;
          },
          [](buffer_t p) { (void)hipFree(p); }));
    }
    return state;
  });
  return ctx;
}

}  // namespace gpu

// ------------------------------------------------------------ host (cpu device) memory
// A program compiled for the gpu keeps its host-placed values (shape tensors, scalars) in
// memory it takes from the cpu device's driver entries
// (R context/base/cpu/cpu_context_impl.cc:105-213; names R device/cpu/cpu_driver.cc:29-35).
namespace gpu {
const char* kRalBaseCpuContextState = "ral_base_cpu_context_state";

void BaseHostContextState::onContextFinish(Context*) {
  std::lock_guard<std::mutex> guard(mu);
  for (const_buffer_t b : host_persistent_buffers) std::free(const_cast<buffer_t>(b));
  host_persistent_buffers.clear();
}

namespace cpu {
namespace {
buffer_t hostAlloc(size_t bytes) {
  // 64-byte aligned, as the reference's aligned_malloc
  const size_t n = (std::max<size_t>(bytes, 1) + 63) / 64 * 64;
  return std::aligned_alloc(64, n);
}
}  // namespace

buffer_t ral_base_cpu_alloc(ExecutionContext* ctx, size_t bytes) {
  auto* exec = dynamic_cast<BaseHipExecutionContext*>(ctx);
  if (!exec) {
    ctx->signalError(Context::FAILURE, "alloc (cpu) needs a BaseHipExecutionContext");
    return nullptr;
  }
  buffer_t ptr = hostAlloc(bytes);
  if (!ptr) {
    ctx->signalError(Context::FAILURE, "host allocation of " + std::to_string(bytes) + " bytes failed");
    return nullptr;
  }
  exec->host_ptr_map[ptr] = 1;
  return ptr;
}

buffer_t ral_base_cpu_alloc_persistent(ExecutionContext* ctx, size_t bytes) {
  auto* state = ctx->getResource<BaseHostContextState>(kRalBaseCpuContextState);
  if (!state) {
    ctx->signalError(Context::FAILURE, "no host memory state in this context");
    return nullptr;
  }
  buffer_t ptr = hostAlloc(bytes);
  if (!ptr) {
    ctx->signalError(Context::FAILURE, "host allocation of " + std::to_string(bytes) + " bytes failed");
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(state->mu);
  state->host_persistent_buffers.insert(ptr);
  return ptr;
}

void ral_base_cpu_dealloc(ExecutionContext* ctx, buffer_t buffer) {
  if (!buffer) return;
  auto* state = ctx->getResource<BaseHostContextState>(kRalBaseCpuContextState);
  if (state) {
    std::lock_guard<std::mutex> guard(state->mu);
    if (state->host_persistent_buffers.count(buffer)) return;   // persistent: ignored
  }
  auto* exec = dynamic_cast<BaseHipExecutionContext*>(ctx);
  if (!exec) return;
  auto it = exec->host_ptr_map.find(buffer);
  if (it == exec->host_ptr_map.end()) return;
  if (--it->second == 0) {
    // (an alias of a program input was pinned by inc_ref: the buffer is the caller's)
    if (!exec->input_ptr_set.count(buffer)) std::free(buffer);
    exec->host_ptr_map.erase(it);
  }
}

buffer_t ral_base_cpu_raw_alloc(Context*, size_t bytes) { return hostAlloc(bytes); }

void ral_base_cpu_raw_dealloc(Context*, buffer_t buffer) { std::free(buffer); }

void ral_base_cpu_memcpy(ExecutionContext*, buffer_t from, buffer_t to, size_t bytes) {
  if (bytes) std::memcpy(to, from, bytes);
}

void ral_base_cpu_memset(ExecutionContext*, buffer_t buffer, int value, size_t bytes) {
  if (bytes) std::memset(buffer, value, bytes);
}

}  // namespace cpu
}  // namespace gpu

TAO_RAL_API("alloc", "cpu", gpu::cpu::ral_base_cpu_alloc);
TAO_RAL_API("ral_cpu_alloc_persistent", "cpu", gpu::cpu::ral_base_cpu_alloc_persistent);
TAO_RAL_API("dealloc", "cpu", gpu::cpu::ral_base_cpu_dealloc);
TAO_RAL_API("raw_cpu_alloc", "cpu", gpu::cpu::ral_base_cpu_raw_alloc);
TAO_RAL_API("raw_cpu_dealloc", "cpu", gpu::cpu::ral_base_cpu_raw_dealloc);
TAO_RAL_API("ral_cpu_memcpy", "cpu", gpu::cpu::ral_base_cpu_memcpy);
TAO_RAL_API("ral_cpu_memset", "cpu", gpu::cpu::ral_base_cpu_memset);

TAO_RAL_API(tao::ral::gpu::kRalGpuAlloc, "gpu", gpu::ral_base_hip_alloc);
TAO_RAL_API(tao::ral::gpu::kRalGpuAllocPersistent, "gpu", gpu::ral_base_hip_alloc_persistent);
TAO_RAL_API(tao::ral::gpu::kRalGpuDealloc, "gpu", gpu::ral_base_hip_dealloc);
TAO_RAL_API(tao::ral::gpu::kRalGpuRawAlloc, "gpu", gpu::ral_base_hip_raw_alloc);
TAO_RAL_API(tao::ral::gpu::kRalGpuRawDealloc, "gpu", gpu::ral_base_hip_raw_dealloc);
TAO_RAL_API(tao::ral::gpu::kRalGpuLaunch, "gpu", gpu::ral_base_hip_launch);
TAO_RAL_API(tao::ral::gpu::kRalGpuGetStream, "gpu", gpu::ral_base_hip_get_stream);
TAO_RAL_API(tao::ral::gpu::kRalGpuAsCUStream, "gpu", gpu::ral_base_hip_as_cu_stream);
TAO_RAL_API(tao::ral::gpu::kRalGpuAsSEStream, "gpu", gpu::ral_base_hip_as_se_stream);
TAO_RAL_API(tao::ral::gpu::kRalGpuH2D, "gpu", gpu::ral_base_hip_h2d);
TAO_RAL_API(tao::ral::gpu::kRalGpuD2H, "gpu", gpu::ral_base_hip_d2h);
TAO_RAL_API(tao::ral::gpu::kRalGpuD2D, "gpu", gpu::ral_base_hip_d2d);
TAO_RAL_API(tao::ral::gpu::kRalGpuSyncOnStream, "gpu", gpu::ral_base_hip_sync_on_stream);
TAO_RAL_API(tao::ral::gpu::kRalGpuSyncAll, "gpu", gpu::ral_base_hip_sync_all);
TAO_RAL_API(tao::ral::gpu::kRalGpuMemset, "gpu", gpu::ral_base_hip_memset);

}  // namespace ral
}  // namespace tao
