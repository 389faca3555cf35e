#include "mlir/ral/device/gpu/gpu_driver.h"

#include <functional>

#include "mlir/ral/ral_context.h"
#include "mlir/ral/ral_helper.h"

namespace tao {
namespace ral {
namespace gpu {

const char* kRalGpuAlloc = "alloc";
const char* kRalGpuAllocPersistent = "ral_gpu_alloc_persistent";
const char* kRalGpuDealloc = "dealloc";
const char* kRalGpuRawAlloc = "raw_gpu_alloc";
const char* kRalGpuRawDealloc = "raw_gpu_dealloc";
const char* kRalGpuD2D = "d2d_";
const char* kRalGpuD2H = "d2h_";
const char* kRalGpuH2D = "h2d_";
const char* kRalGpuMemset = "ral_gpu_memset";
const char* kRalGpuLaunch = "ral_kernel_launch";
const char* kRalGpuGetStream = "ral_gpu_get_stream";
const char* kRalGpuSyncOnStream = "sync_on_stream";
const char* kRalGpuSyncAll = "ral_gpu_sync_all";
const char* kRalGpuAsCUStream = "ral_gpu_as_cu_stream";
const char* kRalGpuAsSEStream = "ral_gpu_as_se_stream";

struct GPUDriver::Impl {
  Context* context = nullptr;
  using E = ExecutionContext*;
  std::function<buffer_t(E, size_t)> alloc;
  std::function<buffer_t(E, size_t)> alloc_persistent;
  std::function<void(E, buffer_t)> dealloc;
  std::function<buffer_t(Context*, size_t)> raw_alloc;
  std::function<void(Context*, buffer_t)> raw_dealloc;
  std::function<void(E, stream_t, buffer_t, buffer_t, size_t)> d2d;
  std::function<void(E, stream_t, buffer_t, buffer_t, size_t)> d2h;
  std::function<void(E, stream_t, const void*, buffer_t, size_t)> h2d;
  std::function<void(E, stream_t, buffer_t, int, size_t)> memset;
  std::function<stream_t(E, int)> getStream;
  std::function<void(E, void**, size_t, const char*, intptr_t, intptr_t, intptr_t,
                     intptr_t, intptr_t, intptr_t, int32_t, stream_t, int32_t, void**)>
      launchKernel;
  std::function<void(E, stream_t)> syncOnStream;
  std::function<void(E)> syncAll;
  std::function<opaque_t(E, stream_t)> asCUStream;
  std::function<opaque_t(E, stream_t)> asSEStream;

  // `alloc` and `dealloc` are shared names between devices, so they are looked up
  // by their full gpu signature; the rest have device-unique bare names.
  template <typename Fn>
  void bindMangled(Fn& slot, const char* bare) {
    slot = DriverApiWrapper<Fn>::Wrapper(context->find(
        TaoRalApiFuncNameHelper<Fn>::Invoke(std::string(bare) + "___gpu")));
  }
  template <typename Fn>
  void bindBare(Fn& slot, const char* bare) {
    slot = DriverApiWrapper<Fn>::Wrapper(context->find(bare));
  }

  void missing(const char* what) {
    context->signalError(Context::FAILURE, std::string(what) + " not implemented");
  }
};

GPUDriver::GPUDriver(Context* context) : impl_(new Impl) {
  impl_->context = context;
  impl_->bindMangled(impl_->alloc, kRalGpuAlloc);
  impl_->bindMangled(impl_->dealloc, kRalGpuDealloc);
  impl_->bindBare(impl_->alloc_persistent, kRalGpuAllocPersistent);
  impl_->bindBare(impl_->raw_alloc, kRalGpuRawAlloc);
  impl_->bindBare(impl_->raw_dealloc, kRalGpuRawDealloc);
  impl_->bindBare(impl_->d2d, kRalGpuD2D);
  impl_->bindBare(impl_->d2h, kRalGpuD2H);
  impl_->bindBare(impl_->h2d, kRalGpuH2D);
  impl_->bindBare(impl_->memset, kRalGpuMemset);
  impl_->bindBare(impl_->launchKernel, kRalGpuLaunch);
  impl_->bindBare(impl_->getStream, kRalGpuGetStream);
  impl_->bindBare(impl_->syncOnStream, kRalGpuSyncOnStream);
  impl_->bindBare(impl_->syncAll, kRalGpuSyncAll);
  impl_->bindBare(impl_->asCUStream, kRalGpuAsCUStream);
  impl_->bindBare(impl_->asSEStream, kRalGpuAsSEStream);
}

GPUDriver::~GPUDriver() = default;

std::string GPUDriver::name() { return "GPUDriver"; }

buffer_t GPUDriver::alloc(ExecutionContext* ctx, size_t bytes) {
  if (!impl_->alloc) return impl_->missing(kRalGpuAlloc), nullptr;
  return impl_->alloc(ctx, bytes);
}

buffer_t GPUDriver::alloc_persistent(ExecutionContext* ctx, size_t bytes) {
  if (!impl_->alloc_persistent) return impl_->missing(kRalGpuAllocPersistent), nullptr;
  return impl_->alloc_persistent(ctx, bytes);
}

void GPUDriver::dealloc(ExecutionContext* ctx, buffer_t buffer) {
  if (!impl_->dealloc) return impl_->missing(kRalGpuDealloc);
  impl_->dealloc(ctx, buffer);
}

buffer_t GPUDriver::raw_alloc(Context* ctx, size_t bytes) {
  if (!impl_->raw_alloc) return impl_->missing(kRalGpuRawAlloc), nullptr;
  return impl_->raw_alloc(ctx, bytes);
}

void GPUDriver::raw_dealloc(Context* ctx, buffer_t buffer) {
  if (!impl_->raw_dealloc) return impl_->missing(kRalGpuRawDealloc);
  impl_->raw_dealloc(ctx, buffer);
}

void GPUDriver::d2d(ExecutionContext* ctx, stream_t s, buffer_t from, buffer_t to,
                    size_t bytes) {
  if (!impl_->d2d) return impl_->missing(kRalGpuD2D);
  impl_->d2d(ctx, s, from, to, bytes);
}

void GPUDriver::d2h(ExecutionContext* ctx, stream_t s, buffer_t from, buffer_t to,
                    size_t bytes) {
  if (!impl_->d2h) return impl_->missing(kRalGpuD2H);
  impl_->d2h(ctx, s, from, to, bytes);
}

void GPUDriver::h2d(ExecutionContext* ctx, stream_t s, const_buffer_t from, buffer_t to,
                    size_t bytes) {
  if (!impl_->h2d) return impl_->missing(kRalGpuH2D);
  impl_->h2d(ctx, s, from, to, bytes);
}

void GPUDriver::memset(ExecutionContext* ctx, stream_t s, buffer_t buffer, int value,
                       size_t bytes) {
  if (!impl_->memset) return impl_->missing(kRalGpuMemset);
  impl_->memset(ctx, s, buffer, value, bytes);
}

stream_t GPUDriver::getStream(ExecutionContext* ctx, int idx) {
  if (!impl_->getStream) return impl_->missing(kRalGpuGetStream), nullptr;
  return impl_->getStream(ctx, idx);
}

void GPUDriver::launchKernel(ExecutionContext* ctx, void** blobs, size_t num_blobs,
                             const char* kernel_name, intptr_t gridX, intptr_t gridY,
                             intptr_t gridZ, intptr_t blockX, intptr_t blockY,
                             intptr_t blockZ, int32_t smem, stream_t stream,
                             int32_t num_args, void** params) {
  if (!impl_->launchKernel) return impl_->missing(kRalGpuLaunch);
  impl_->launchKernel(ctx, blobs, num_blobs, kernel_name, gridX, gridY, gridZ, blockX,
                      blockY, blockZ, smem, stream, num_args, params);
}

void GPUDriver::syncOnStream(ExecutionContext* ctx, stream_t s) {
  if (!impl_->syncOnStream) return impl_->missing(kRalGpuSyncOnStream);
  impl_->syncOnStream(ctx, s);
}

void GPUDriver::syncAll(ExecutionContext* ctx) {
  if (!impl_->syncAll) return impl_->missing(kRalGpuSyncAll);
  impl_->syncAll(ctx);
}

opaque_t GPUDriver::asCUStream(ExecutionContext* ctx, stream_t s) {
  if (!impl_->asCUStream) return impl_->missing(kRalGpuAsCUStream), nullptr;
  return impl_->asCUStream(ctx, s);
}

opaque_t GPUDriver::asSEStream(ExecutionContext* ctx, stream_t s) {
  if (!impl_->asSEStream) return impl_->missing(kRalGpuAsSEStream), nullptr;
  return impl_->asSEStream(ctx, s);
}

}  // namespace gpu
}  // namespace ral
}  // namespace tao
