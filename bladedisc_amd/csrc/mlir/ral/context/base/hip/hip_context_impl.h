// The concrete RAL context for one AMD GPU: device memory with a size-class pool,
// one hipStream_t for every copy and launch, and the gpu driver function set
// registered under the names GPUDriver resolves.  Counterpart of the reference's
// tao_compiler/mlir/ral/context/base/cuda/cuda_context_impl.{h,cc} (options :52-60,
// driver functions :258-510, registrations :746-764) and of
// context/base/base_context.{h,cc} (BaseContext, InternalAllocator).
#ifndef RAL_CONTEXT_BASE_HIP_HIP_CONTEXT_IMPL_H_
#define RAL_CONTEXT_BASE_HIP_HIP_CONTEXT_IMPL_H_

#include <hip/hip_runtime.h>

#include <map>
#include <memory>
#include <string>
#include <mutex>
#include <unordered_map>
#include <unordered_set>
#include <utility>
#include <vector>

#include "mlir/ral/device/gpu/gpu_driver.h"
#include "mlir/ral/ral_base.h"
#include "mlir/ral/ral_context.h"
#include "mlir/ral/ral_metadata.h"

namespace tao {
namespace ral {

struct BaseContextOption {
  // Path of the compiled program's constant store.  Empty is allowed: kernels can
  // then be exercised without a compiled model.
  std::string metadata_file_path;
  bool cache_workspace_mem_across_execution = false;
};

class BaseContext : public Context {
 public:
  explicit BaseContext(BaseContextOption& opt);
  ~BaseContext() override;
  const BaseContextOption& option() const { return opt_; }

 private:
  BaseContextOption opt_;
};

// Pooling allocator on top of a raw alloc/dealloc pair.  Requests are rounded up
// to a size class (four classes per power of two, so at most 25 % slack) and freed
// blocks are kept per class: with a dynamic M every call asks for a different byte
// count, and exact-size free lists would never hit.
class InternalAllocator : public Allocator {
 public:
  InternalAllocator(alloc_t alloc_func, dealloc_t dealloc_func);
  ~InternalAllocator() override;

  void releaseAllFreeBuffers() override;
  buffer_t alloc(size_t bytes) override;
  void dealloc(buffer_t buffer) override;

  static size_t sizeClass(size_t bytes);
  size_t liveBytes() const { return live_bytes_; }
  size_t pooledBytes() const { return pooled_bytes_; }

 private:
  alloc_t alloc_func_;
  dealloc_t dealloc_func_;
  std::map<size_t, std::vector<buffer_t>> free_by_class_;
  std::unordered_map<buffer_t, size_t> class_of_;
  size_t live_bytes_ = 0;
  size_t pooled_bytes_ = 0;
};

namespace gpu {

using GpuStreamHandle = hipStream_t;

struct BaseHipContextOption {
  GpuStreamHandle stream = nullptr;  // nullptr = the null stream
  int device_ordinal = 0;
  // e.g. the embedding framework's caching allocator; nullptr = hipMalloc + pool
  std::shared_ptr<Allocator> gpu_allocator;
};

std::unique_ptr<BaseContext> MakeBaseHipContext(BaseContextOption& opt,
                                                BaseHipContextOption& gpu_opt);

// A program output as handed to the embedding framework.  When the wrapper owns the
// buffer (the program allocated it and nothing else refers to it) its destructor
// returns the buffer to the context's allocator, unless release() was called first.
class BaseOutputBufferWrapper : public OutputBufferWrapper {
 public:
  using Deleter = std::function<void(buffer_t)>;
  BaseOutputBufferWrapper(buffer_t data, buffer_shape_t shape)
      : data_(data), shape_(std::move(shape)) {}
  ~BaseOutputBufferWrapper() override {
    if (deleter_) deleter_(data_);
  }
  const_buffer_t data() override { return data_; }
  const buffer_shape_t& shape() override { return shape_; }
  void set_deleter(Deleter deleter) { deleter_ = std::move(deleter); }
  bool owned() const override { return owned_; }
  void markOwned() override { owned_ = true; }
  void release() override {
    deleter_ = nullptr;
    owned_ = false;
  }

 private:
  buffer_t data_;
  buffer_shape_t shape_;
  Deleter deleter_;
  bool owned_ = false;
};

struct Tensor {
  buffer_t buffer = nullptr;
  buffer_shape_t shape;
};

// One run of a compiled program: its input / output bindings and the buffers it
// allocated.  Counterpart of BaseExecutionContext + BaseCudaExecutionContext
// (context/base/base_context.cc:63-95, context/base/cuda/cuda_context_impl.cc:219-252).
struct BaseHipExecutionContext : public ExecutionContext {
  explicit BaseHipExecutionContext(BaseContext* ctx);
  ~BaseHipExecutionContext() override;

  void bindInput(int input_idx, buffer_t buffer, const buffer_shape_t& shape) override;
  void bindOutput(int output_idx, std::unique_ptr<OutputBufferWrapper>* output) override;

  // buffers handed out by `alloc` during this execution -> reference count
  std::unordered_map<const_buffer_t, int> device_ptr_map;
  // the same for host buffers (`alloc` of the cpu device: shape tensors and other host-placed
  // values of a program compiled for the gpu)
  std::unordered_map<const_buffer_t, int> host_ptr_map;
  std::unordered_map<int32_t, Tensor> inputs;
  std::unordered_map<int32_t, Tensor> outputs;
  std::unordered_set<const_buffer_t> input_ptr_set;
  std::unordered_set<const_buffer_t> output_ptr_set;
  // how many outputs share one underlying buffer
  std::unordered_map<const_buffer_t, int32_t> outputSharedOrder;
};

extern const char* kRalBaseHipContextState;

// Host memory of the cpu-device driver entries (reference: ral/context/base/cpu/
// cpu_context_impl.cc:105-204, BaseCpuContextState): buffers that outlive executions.
struct BaseHostContextState : public Context::Resource {
  std::mutex mu;
  std::unordered_set<const_buffer_t> host_persistent_buffers;
  void onContextFinish(Context* ctx) override;
};
extern const char* kRalBaseCpuContextState;

// Context-level store of the program's constants (ral_const): loaded lazily from the
// metadata file named in BaseContextOption, kept for the life of the context.
struct ProcessLevelConstStore;
struct RalGlobalConstantState : public Context::Resource {
  using Item = std::pair<buffer_t, buffer_shape_t>;
  std::mutex mu;
  std::unordered_map<std::string, Item> host_constants;
  std::unordered_map<std::string, Item> device_constants;
  // addresses of the device constants above (what isPersistentDeviceBuffer consults for the
  // process-level store, whose buffers belong to no context's allocator)
  std::unordered_set<const_buffer_t> device_constant_buffers;
  std::unique_ptr<MetadataFile> metadata;
  // if set, the constants live in this store, shared by every context of the process that was
  // made from the same metadata file, instead of in the maps above
  ProcessLevelConstStore* process_level_store = nullptr;
  void onContextFinish(Context* ctx) override;
};
extern const char* kRalGlobalConstantState;

// Process-level store of constants (reference: ral/context/common_context_impl.h:34-58,
// 116-119; common_context_impl.cc:152-186): one per metadata file path, reference-counted by
// the contexts that use it; its device buffers are released by the last context to finish
// (the reference takes them from raw_alloc, i.e. from the embedding framework's allocator,
// which outlives its contexts; here they come straight from hipMalloc).  Switched on by DISC_USE_GLOBAL_CONST_STORE=true|1
// (common_context_impl.cc:57-64, read once per process).
struct ProcessLevelConstStore {
  RalGlobalConstantState state;
  std::string pb_file_path;
};
struct ConstStoreRegistrar {
  static ConstStoreRegistrar& Instance();
  // true if the caller was the last user and now owns (and must release) the store
  bool unregisterConstStore(ProcessLevelConstStore* store);
  ProcessLevelConstStore* getConstStore(const std::string& pb_file_path);
  std::mutex mu;
  std::unordered_map<std::string, ProcessLevelConstStore*> pbFile2Instance;
  std::unordered_map<ProcessLevelConstStore*, int> referenceCounter;
};
bool discEnableGlobalConstantStore();
// Device memory of the process-level store: owned by no context (a context's own allocator
// returns everything it handed out when the context goes away, and these buffers must
// outlive all but the last of their users).
buffer_t processLevelDeviceAlloc(size_t bytes);
void processLevelDeviceFree(buffer_t buffer);

// device buffers that outlive executions (alloc_persistent, and the constants of the
// process-level store): true if `buffer` is one
bool isPersistentDeviceBuffer(ExecutionContext* ctx, const_buffer_t buffer);

}  // namespace gpu
}  // namespace ral
}  // namespace tao

#endif  // RAL_CONTEXT_BASE_HIP_HIP_CONTEXT_IMPL_H_
