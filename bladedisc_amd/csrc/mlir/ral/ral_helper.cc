#include "mlir/ral/ral_helper.h"

#include <algorithm>
#include <mutex>
#include <unordered_map>

#include "mlir/ral/ral_logging.h"

namespace tao {
namespace ral {

struct TaoRalApiRegistry::Impl {
  std::mutex mu;
  std::unordered_map<std::string, api_func_t> table;
};

TaoRalApiRegistry::TaoRalApiRegistry() : impl_(new Impl) {}
TaoRalApiRegistry::~TaoRalApiRegistry() = default;

TaoRalApiRegistry& TaoRalApiRegistry::Global() {
  // function-local static: usable from other translation units' static
  // initialisers (that is how TAO_RAL_API registers)
  static TaoRalApiRegistry instance;
  return instance;
}

bool TaoRalApiRegistry::Register(const std::string& name, const std::string& nickname,
                                 api_func_t api_func) {
  std::lock_guard<std::mutex> guard(impl_->mu);
  const bool fresh = impl_->table.emplace(name, api_func).second;
  TAO_VLOG(1) << "register ral function: " << name << (fresh ? "" : " (duplicate ignored)");
  // the first overload registered under a bare name keeps it
  impl_->table.emplace(nickname, api_func);
  return fresh;
}

TaoRalApiRegistry::api_func_t TaoRalApiRegistry::Find(const std::string& name) {
  std::lock_guard<std::mutex> guard(impl_->mu);
  auto it = impl_->table.find(name);
  return it == impl_->table.end() ? api_func_t() : it->second;
}

std::vector<std::string> TaoRalApiRegistry::Names() {
  std::vector<std::string> out;
  {
    std::lock_guard<std::mutex> guard(impl_->mu);
    out.reserve(impl_->table.size());
    for (auto& kv : impl_->table) out.push_back(kv.first);
  }
  std::sort(out.begin(), out.end());
  return out;
}

}  // namespace ral
}  // namespace tao
