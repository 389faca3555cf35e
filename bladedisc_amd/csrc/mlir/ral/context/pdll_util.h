// Attributes of ral_pdll_* custom calls.  The compiler serialises the call's
// `custom_attrs` dictionary into a byte blob (writer: the reference's
// disc/transforms/disc_lower_to_library_call.cc:684-848) and passes its address as
// the last `void*` argument; this is the reader.  Class names and accessors follow
// the reference's tao_compiler/mlir/ral/context/pdll_util.h:27-221.
//
// Wire format (host endian, recursive):
//   string  := int64 length, bytes
//   attr    := string type-tag, payload
//   "dict"  : int64 n, n x (string key, attr)
//   "str"   : string
//   "bool"  : 1 byte          "int": int64          "float": double
//   "intArray": int64 n, n x int64        "array": int64 n, n x attr
//   "denseElementsAttr": string elem kind ("int"|"uint"|"float"), unsigned bits,
//                        int64 rank, rank x int64 dims, 1 byte splat, string raw data
#ifndef RAL_CONTEXT_PDLL_UTIL_H_
#define RAL_CONTEXT_PDLL_UTIL_H_

#include <cassert>
#include <cstdint>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "mlir/ral/ral_context.h"

namespace tao {
namespace ral {

class PDLAttr {
 public:
  explicit PDLAttr(const std::string& type) : type_(type) {}
  virtual ~PDLAttr() {}
  const std::string& getType() const { return type_; }

  // Unchecked downcast, as in the reference; check getType() when in doubt.
  template <typename T>
  T& as() {
    return *static_cast<T*>(this);
  }

 private:
  std::string type_;
};

using PDLAttrPtr = std::unique_ptr<PDLAttr>;

class StrPDLAttr : public PDLAttr {
 public:
  StrPDLAttr(const std::string& type, const std::string& str) : PDLAttr(type), str_(str) {}
  std::string& getValue() { return str_; }

 private:
  std::string str_;
};

template <typename T>
class PodPDLAttr : public PDLAttr {
 public:
  PodPDLAttr(const std::string& type, T val) : PDLAttr(type), val_(val) {}
  T getValue() { return val_; }

 private:
  T val_;
};

using BoolPDLAttr = PodPDLAttr<bool>;
using IntPDLAttr = PodPDLAttr<int64_t>;
using FloatPDLAttr = PodPDLAttr<double>;

class DenseElementsPDLAttr : public PDLAttr {
 public:
  DenseElementsPDLAttr(const std::string& type, const std::string& elemTy, unsigned numBits,
                       std::vector<int64_t> shape, std::vector<uint8_t> rawData)
      : PDLAttr(type), elemTy_(elemTy), numBits_(numBits), shape_(std::move(shape)),
        rawData_(std::move(rawData)) {}

  std::vector<uint8_t>& getRawData() { return rawData_; }
  template <typename T>
  T* getValue() {
    return reinterpret_cast<T*>(rawData_.data());
  }
  std::vector<int64_t> getShape() { return shape_; }
  const std::string& getElementType() { return elemTy_; }
  unsigned getNumBits() { return numBits_; }
  int64_t getNumElements() {
    int64_t n = 1;
    for (int64_t d : shape_) n *= d;
    return n;
  }

 private:
  std::string elemTy_;
  unsigned numBits_;
  std::vector<int64_t> shape_;
  std::vector<uint8_t> rawData_;
};

class DictPDLAttr : public PDLAttr {
 public:
  using PDLAttr::PDLAttr;
  bool hasKey(const std::string& key) const { return items_.count(key) != 0; }
  // The key must exist (check hasKey first when it is optional).
  PDLAttr& get(const std::string& key) {
    auto it = items_.find(key);
    assert(it != items_.end());
    return *it->second;
  }
  bool insert(const std::string& key, PDLAttrPtr value) {
    return items_.emplace(key, std::move(value)).second;
  }
  std::unordered_map<std::string, PDLAttrPtr>& getValue() { return items_; }

 private:
  std::unordered_map<std::string, PDLAttrPtr> items_;
};

class ArrayPDLAttr : public PDLAttr {
 public:
  using PDLAttr::PDLAttr;
  PDLAttr& get(int64_t index) { return *items_.at(index); }
  uint64_t size() { return items_.size(); }
  void push_back(PDLAttrPtr value) { items_.push_back(std::move(value)); }
  std::vector<PDLAttrPtr>& getValue() { return items_; }

 private:
  std::vector<PDLAttrPtr> items_;
};

class IntArrayPDLAttr : public PDLAttr {
 public:
  using PDLAttr::PDLAttr;
  int64_t get(int64_t index) { return items_.at(index); }
  uint64_t size() { return items_.size(); }
  void push_back(int64_t v) { items_.push_back(v); }
  std::vector<int64_t>& getValue() { return items_; }

 private:
  std::vector<int64_t> items_;
};

// Parses one attr starting at `buffer` and advances it.  Returns nullptr on an
// unknown type tag or a malformed blob.
std::unique_ptr<PDLAttr> parsePDLAttr(uint8_t*& buffer);
// Same with a known blob size: never reads beyond buffer + size.
std::unique_ptr<PDLAttr> parsePDLAttr(const uint8_t* buffer, size_t size, size_t* consumed);

template <typename T>
struct CustomAttrState : public Context::Resource {
  std::mutex mu;
  std::unordered_map<void*, std::unique_ptr<T>> customAttrMap;
};

// Blobs are constants of the compiled program: parse each once per context and
// key the result by the blob's address.
template <typename T>
inline T* getOrParseCustomAttr(ExecutionContext* ctx, void* attrPtr, const std::string& name,
                               std::function<std::unique_ptr<T>()> creator) {
  using StateTy = CustomAttrState<T>;
  auto* state = ctx->getOrCreateResource<StateTy>(name, [] { return new StateTy; });
  if (!state) return nullptr;
  std::lock_guard<std::mutex> guard(state->mu);
  auto it = state->customAttrMap.find(attrPtr);
  if (it == state->customAttrMap.end()) {
    auto value = creator();
    if (!value) return nullptr;
    it = state->customAttrMap.emplace(attrPtr, std::move(value)).first;
  }
  return it->second.get();
}

inline PDLAttr* getOrParsePDLAttr(ExecutionContext* ctx, void* attrPtr,
                                  const std::string& name) {
  if (!attrPtr) return nullptr;
  return getOrParseCustomAttr<PDLAttr>(ctx, attrPtr, name, [attrPtr] {
    auto* p = static_cast<uint8_t*>(attrPtr);
    return parsePDLAttr(p);
  });
}

}  // namespace ral
}  // namespace tao

#endif  // RAL_CONTEXT_PDLL_UTIL_H_
