// GPU driver facade used by kernels for memory and stream services.  Same interface
// as the reference's tao_compiler/mlir/ral/device/gpu/gpu_driver.h:53-112; every
// method forwards to a function looked up in the RAL registry by name when the
// driver is constructed (reference gpu_driver.cc:27-41,70-113), so an embedding
// framework can replace any of them by registering its own.
#ifndef RAL_GPU_GPU_DRIVER_H_
#define RAL_GPU_GPU_DRIVER_H_

#include <memory>
#include <string>

#include "mlir/ral/ral_driver.h"

namespace tao {
namespace ral {

class Context;
class ExecutionContext;

namespace gpu {

using stream_t = void*;  // a stream *index* cast to a pointer; only 0 exists

extern const char* kRalGpuAlloc;
extern const char* kRalGpuAllocPersistent;
extern const char* kRalGpuDealloc;
extern const char* kRalGpuRawAlloc;
extern const char* kRalGpuRawDealloc;
extern const char* kRalGpuD2D;
extern const char* kRalGpuD2H;
extern const char* kRalGpuH2D;
extern const char* kRalGpuMemset;
extern const char* kRalGpuLaunch;
extern const char* kRalGpuGetStream;
extern const char* kRalGpuSyncOnStream;
extern const char* kRalGpuSyncAll;
extern const char* kRalGpuAsCUStream;
extern const char* kRalGpuAsSEStream;

class GPUDriver : public Driver {
 public:
  explicit GPUDriver(Context* context);
  ~GPUDriver();

  static std::string name();

  // per-execution device memory (ref-counted by the execution context)
  buffer_t alloc(ExecutionContext* ctx, size_t);
  // device memory that outlives executions; released with the context
  buffer_t alloc_persistent(ExecutionContext* ctx, size_t);
  void dealloc(ExecutionContext* ctx, buffer_t);

  // untracked device memory: the caller pairs alloc and dealloc
  buffer_t raw_alloc(Context* ctx, size_t);
  void raw_dealloc(Context* ctx, buffer_t);

  // all copies are asynchronous on the context's stream
  void d2d(ExecutionContext* ctx, stream_t, buffer_t from, buffer_t to, size_t);
  void d2h(ExecutionContext* ctx, stream_t, buffer_t from, buffer_t to, size_t);
  void h2d(ExecutionContext* ctx, stream_t, const_buffer_t from, buffer_t to, size_t);
  void memset(ExecutionContext* ctx, stream_t, buffer_t, int, size_t);

  stream_t getStream(ExecutionContext* ctx, int idx);

  // launches a kernel of a compiler-generated code object
  void launchKernel(ExecutionContext* ctx, void** blobs, size_t num_blobs,
                    const char* kernel_name, intptr_t gridX, intptr_t gridY,
                    intptr_t gridZ, intptr_t blockX, intptr_t blockY, intptr_t blockZ,
                    int32_t smem, stream_t stream, int32_t num_args, void** params);

  void syncOnStream(ExecutionContext* ctx, stream_t);
  void syncAll(ExecutionContext* ctx);

  // the platform stream behind `stream_t`: a hipStream_t here
  opaque_t asCUStream(ExecutionContext* ctx, stream_t);
  // always nullptr: there is no StreamExecutor in this runtime
  opaque_t asSEStream(ExecutionContext* ctx, stream_t);

 private:
  struct Impl;
  std::unique_ptr<Impl> impl_;
};

}  // namespace gpu
}  // namespace ral
}  // namespace tao

#endif  // RAL_GPU_GPU_DRIVER_H_
