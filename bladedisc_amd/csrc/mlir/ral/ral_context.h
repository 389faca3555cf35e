// Context / ExecutionContext / Resource: the state a compiled DISC program runs
// against.  Same public interface as the reference's tao_compiler/mlir/ral/ral_context.h
// (:59-204).  One Context may serve several concurrent ExecutionContexts.
//
// Error model: signalError records the first error and makes every later call()
// return immediately until clearError().  The reference logs at FATAL, i.e. aborts
// the process (ral_context.cc:185-191); set DISC_RAL_ABORT_ON_ERROR=1 for that.
#ifndef RAL_RAL_CONTEXT_H_
#define RAL_RAL_CONTEXT_H_

#include <cstdint>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <type_traits>
#include <unordered_map>
#include <vector>

#include "mlir/ral/ral_base.h"

namespace tao {
namespace ral {

extern const char* kRalRecvInput;
extern const char* kRalSendOutput;
extern const char* kRalCudaConst;
extern const char* kRalHostConst;
extern const char* kRalBitcast;

class Driver;
class ExecutionContext;

struct ThreadLocalIndex {
  // small dense id of the calling thread
  static int Get();
};

class Context {
 public:
  Context();
  virtual ~Context();

  enum { SUCCESS = 0, FAILURE = 1 };

  // Calls the registered function `api_name` with the packed arguments.
  virtual void call(const std::string& api_name, void** args);
  // Same; `api_name` is expected to be a string constant of the compiled program,
  // so the lookup is cached per thread by pointer identity.
  void call(const char* api_name, void** args);

  virtual api_func_t find(const std::string& api_name);

  status_t getLastError(const char** err_msg);
  void signalError(status_t errcode, const std::string& err_msg);
  void clearError();

  virtual void onExecutionStart(ExecutionContext*);
  virtual void onExecutionFinish(ExecutionContext*);

  // State owned by the context and shared by every execution on it.
  struct Resource {
    virtual ~Resource() = default;
    virtual void onExecutionStart(ExecutionContext*) {}
    virtual void onExecutionFinish(ExecutionContext*) {}
    virtual void onContextFinish(Context*) {}
  };

  enum LifetimeKind { kPerContext, kPerExecution, kGlobal };

  // Returns the resource named `key`, creating it with `creator` on first use.
  // Returns nullptr if the context is in error state or creation fails.
  virtual std::shared_ptr<Resource> getOrCreateResource(
      const std::string& key, std::function<Resource*()> creator);

  virtual void addDriver(const std::string& name, std::unique_ptr<Driver> driver);
  virtual Driver* getDriver(const std::string& name);

 protected:
  void signalErrorLocked(status_t errcode, const std::string& err_msg);

  struct Impl;
  std::mutex mu;
  std::unique_ptr<Impl> impl_;
};

class OutputBufferWrapper {
 public:
  virtual ~OutputBufferWrapper() {}
  virtual const_buffer_t data() = 0;
  virtual const buffer_shape_t& shape() = 0;
  virtual bool owned() const = 0;
  virtual void markOwned() = 0;
  virtual void release() = 0;
};

class ExecutionContext {
 public:
  explicit ExecutionContext(Context* context);
  virtual ~ExecutionContext();

  Context* getContext();

  virtual void bindInput(int /*input_idx*/, buffer_t /*buffer*/,
                         const buffer_shape_t& /*shape*/) {}
  virtual void bindOutput(int /*output_idx*/,
                          std::unique_ptr<OutputBufferWrapper>* /*output*/) {}

  template <typename T>
  T* getOrCreateResource(const std::string& key,
                         std::function<Context::Resource*()> creator) {
    auto it = cachedResources_.find(key);
    if (it == cachedResources_.end()) {
      Context::Resource* r = getContext()->getOrCreateResource(key, creator).get();
      if (!r) return nullptr;
      it = cachedResources_.emplace(key, r).first;
    }
    return static_cast<T*>(it->second);
  }

  template <typename T>
  T* getResource(const std::string& key) {
    return getOrCreateResource<T>(key, nullptr);
  }

  void signalError(status_t errcode, const std::string& err_msg) {
    getContext()->signalError(errcode, err_msg);
  }

  template <typename T>
  T* getDriver(const std::string& name) {
    return static_cast<T*>(getContext()->getDriver(name));
  }

  void onExecutionStart() { getContext()->onExecutionStart(this); }
  void onExecutionFinish() { getContext()->onExecutionFinish(this); }

 private:
  Context* context_;
  std::unordered_map<std::string, Context::Resource*> cachedResources_;
};

template <typename T,
          typename = typename std::enable_if<std::is_base_of<ExecutionContext, T>::value>::type,
          typename... Args>
std::unique_ptr<T> MakeExecutionContext(Args&&... args) {
  return std::unique_ptr<T>(new T(std::forward<Args>(args)...));
}

}  // namespace ral
}  // namespace tao

#endif  // RAL_RAL_CONTEXT_H_
