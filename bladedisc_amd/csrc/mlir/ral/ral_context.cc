#include "mlir/ral/ral_context.h"

#include <atomic>
#include <cstdlib>
#include <map>
#include <thread>

#include "mlir/ral/ral_driver.h"
#include "mlir/ral/ral_helper.h"
#include "mlir/ral/ral_logging.h"

namespace tao {
namespace ral {

const char* kRalRecvInput = "ral_recv_input";
const char* kRalSendOutput = "ral_send_output";
const char* kRalCudaConst = "ral_const";
const char* kRalHostConst = "ral_const";
const char* kRalBitcast = "inc_ref";

int ThreadLocalIndex::Get() {
  static std::atomic<int> next{0};
  static thread_local int mine = next.fetch_add(1);
  return mine;
}

namespace {

bool AbortOnError() {
  static const bool v = [] {
    const char* e = std::getenv("DISC_RAL_ABORT_ON_ERROR");
    return e && e[0] && e[0] != '0';
  }();
  return v;
}

// name-pointer -> function cache, one per (thread, context): compiled programs
// pass the same string constant on every call, so a pointer compare suffices.
struct PointerCache {
  std::unordered_map<const char*, api_func_t> by_ptr;
};

std::atomic<uint64_t> g_next_context_id{1};

}  // namespace

struct Context::Impl {
  // never reused, unlike the Context's address: guards the thread-local cache
  // lookup below against a new context allocated where a destroyed one lived
  const uint64_t id = g_next_context_id.fetch_add(1);
  status_t errcode = 0;
  std::string err_msg;
  std::unordered_map<std::string, std::unique_ptr<Driver>> drivers;
  // ordered: hooks run in a deterministic order
  std::map<std::string, std::shared_ptr<Resource>> resources;

  std::mutex cache_mu;
  std::unordered_map<int, std::unique_ptr<PointerCache>> caches;  // by thread index

  PointerCache* cacheForThisThread() {
    const int tid = ThreadLocalIndex::Get();
    std::lock_guard<std::mutex> guard(cache_mu);
    auto& slot = caches[tid];
    if (!slot) slot.reset(new PointerCache);
    return slot.get();
  }
};

Context::Context() : impl_(new Impl) {}

Context::~Context() {
  for (auto& kv : impl_->resources) kv.second->onContextFinish(this);
}

void Context::call(const std::string& api_name, void** args) {
  {
    std::lock_guard<std::mutex> guard(mu);
    if (impl_->errcode != 0) return;  // an earlier error poisons later calls
  }
  api_func_t fn = find(api_name);
  if (!fn) {
    if (api_name.compare(0, 9, "ral_debug") == 0) {
      TAO_VLOG(0) << "[[DEBUG]] " << api_name;
      return;
    }
    signalError(FAILURE, "api_func " + api_name + " not found");
    return;
  }
  TAO_VLOG(1) << "call api_func " << api_name;
  fn(args);
}

void Context::call(const char* api_name, void** args) {
  {
    std::lock_guard<std::mutex> guard(mu);
    if (impl_->errcode != 0) return;
  }
  // each thread only touches its own cache object after the locked lookup
  static thread_local uint64_t cached_for = 0;
  static thread_local PointerCache* cache = nullptr;
  if (cached_for != impl_->id) {
    cache = impl_->cacheForThisThread();
    cached_for = impl_->id;
  }
  auto it = cache->by_ptr.find(api_name);
  if (it == cache->by_ptr.end()) {
    api_func_t fn = find(std::string(api_name));
    if (!fn) {
      signalError(FAILURE, "api_func " + std::string(api_name) + " not found");
      return;
    }
    it = cache->by_ptr.emplace(api_name, std::move(fn)).first;
  }
  TAO_VLOG(1) << "call api_func " << api_name;
  it->second(args);
}

api_func_t Context::find(const std::string& api_name) {
  return TaoRalApiRegistry::Global().Find(api_name);
}

void Context::onExecutionStart(ExecutionContext* exec_ctx) {
  std::lock_guard<std::mutex> guard(mu);
  for (auto& kv : impl_->resources) kv.second->onExecutionStart(exec_ctx);
}

void Context::onExecutionFinish(ExecutionContext* exec_ctx) {
  std::lock_guard<std::mutex> guard(mu);
  for (auto& kv : impl_->resources) kv.second->onExecutionFinish(exec_ctx);
}

status_t Context::getLastError(const char** msg_ptr) {
  // the message is copied into thread-local storage: another thread may change
  // the context's status while the caller still reads the string
  static thread_local std::string local_msg;
  std::lock_guard<std::mutex> guard(mu);
  if (msg_ptr) {
    local_msg = impl_->err_msg;
    *msg_ptr = local_msg.c_str();
  }
  return impl_->errcode;
}

void Context::signalError(status_t errcode, const std::string& err_msg) {
  if (errcode == 0) return;
  std::lock_guard<std::mutex> guard(mu);
  signalErrorLocked(errcode, err_msg);
}

void Context::clearError() {
  std::lock_guard<std::mutex> guard(mu);
  impl_->errcode = 0;
  impl_->err_msg.clear();
}

void Context::signalErrorLocked(status_t errcode, const std::string& err_msg) {
  if (AbortOnError()) {
    TAO_LOG(FATAL) << "[[ERROR]] Context catch an exception: " << err_msg;
  }
  TAO_LOG(ERROR) << "[[ERROR]] Context catch an exception: " << err_msg;
  if (impl_->errcode == 0) {  // keep the first error
    impl_->errcode = errcode;
    impl_->err_msg = err_msg;
  }
}

void Context::addDriver(const std::string& name, std::unique_ptr<Driver> driver) {
  std::lock_guard<std::mutex> guard(mu);
  impl_->drivers.emplace(name, std::move(driver));  // an existing driver wins
}

Driver* Context::getDriver(const std::string& name) {
  std::lock_guard<std::mutex> guard(mu);
  auto it = impl_->drivers.find(name);
  return it == impl_->drivers.end() ? nullptr : it->second.get();
}

std::shared_ptr<Context::Resource> Context::getOrCreateResource(
    const std::string& key, std::function<Resource*()> creator) {
  std::lock_guard<std::mutex> guard(mu);
  if (impl_->errcode != 0) return nullptr;
  auto it = impl_->resources.find(key);
  if (it != impl_->resources.end()) return it->second;
  Resource* fresh = creator ? creator() : nullptr;
  if (!fresh) {
    signalErrorLocked(FAILURE, "resource creation failed: " + key);
    return nullptr;
  }
  return impl_->resources.emplace(key, std::shared_ptr<Resource>(fresh)).first->second;
}

ExecutionContext::ExecutionContext(Context* context) : context_(context) {}
ExecutionContext::~ExecutionContext() = default;
Context* ExecutionContext::getContext() { return context_; }

}  // namespace ral
}  // namespace tao
