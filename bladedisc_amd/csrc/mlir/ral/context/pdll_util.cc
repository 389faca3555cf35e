#include "mlir/ral/context/pdll_util.h"

#include <cstring>
#include <limits>

namespace tao {
namespace ral {
namespace {

// Bounds-checked cursor over the blob.
class Reader {
 public:
  Reader(const uint8_t* p, size_t size) : p_(p), left_(size) {}

  template <typename T>
  bool pod(T* out) {
    if (left_ < sizeof(T)) return false;
    std::memcpy(out, p_, sizeof(T));  // blobs are byte strings: no alignment promise
    p_ += sizeof(T);
    left_ -= sizeof(T);
    return true;
  }

  bool str(std::string* out) {
    int64_t n = 0;
    if (!pod(&n) || n < 0 || static_cast<uint64_t>(n) > left_) return false;
    out->assign(reinterpret_cast<const char*>(p_), static_cast<size_t>(n));
    p_ += n;
    left_ -= static_cast<size_t>(n);
    return true;
  }

  const uint8_t* pos() const { return p_; }

 private:
  const uint8_t* p_;
  size_t left_;
};

constexpr int kMaxDepth = 64;
constexpr int64_t kMaxCount = int64_t(1) << 32;

PDLAttrPtr parseAny(Reader& r, int depth);

PDLAttrPtr parseDict(Reader& r, const std::string& tag, int depth) {
  int64_t n = 0;
  if (!r.pod(&n) || n < 0 || n > kMaxCount) return nullptr;
  auto dict = std::make_unique<DictPDLAttr>(tag);
  for (int64_t i = 0; i < n; ++i) {
    std::string key;
    if (!r.str(&key)) return nullptr;
    PDLAttrPtr value = parseAny(r, depth + 1);
    if (!value) return nullptr;
    dict->insert(key, std::move(value));
  }
  return dict;
}

PDLAttrPtr parseDense(Reader& r, const std::string& tag) {
  std::string elem;
  unsigned bits = 0;
  int64_t rank = 0;
  if (!r.str(&elem) || !r.pod(&bits) || !r.pod(&rank) || rank < 0 || rank > 64)
    return nullptr;
  std::vector<int64_t> shape;
  int64_t count = 1;
  for (int64_t i = 0; i < rank; ++i) {
    int64_t d = 0;
    if (!r.pod(&d) || d < 0) return nullptr;
    shape.push_back(d);
    if (d != 0 && count > kMaxCount / d) return nullptr;
    count *= d;
  }
  uint8_t splat_byte = 0;   // read as a byte: any non-zero value means "splat"
  std::string raw;
  if (!r.pod(&splat_byte) || !r.str(&raw)) return nullptr;
  const bool splat = splat_byte != 0;
  std::vector<uint8_t> data(raw.begin(), raw.end());
  if (splat) {
    // one element stored; expand it to the full shape
    const size_t width = bits / 8;
    if (width == 0 || data.size() != width) return nullptr;
    std::vector<uint8_t> full(static_cast<size_t>(count) * width);
    for (size_t i = 0; i < full.size(); ++i) full[i] = data[i % width];
    data.swap(full);
  }
  return std::make_unique<DenseElementsPDLAttr>(tag, elem, bits, std::move(shape),
                                                std::move(data));
}

PDLAttrPtr parseAny(Reader& r, int depth) {
  if (depth > kMaxDepth) return nullptr;
  std::string tag;
  if (!r.str(&tag)) return nullptr;
  if (tag == "dict") return parseDict(r, tag, depth);
  if (tag == "str") {
    std::string v;
    if (!r.str(&v)) return nullptr;
    return std::make_unique<StrPDLAttr>(tag, v);
  }
  if (tag == "bool") {
    uint8_t v = 0;
    if (!r.pod(&v)) return nullptr;
    return std::make_unique<BoolPDLAttr>(tag, v != 0);
  }
  if (tag == "int") {
    int64_t v = 0;
    if (!r.pod(&v)) return nullptr;
    return std::make_unique<IntPDLAttr>(tag, v);
  }
  if (tag == "float") {
    double v = 0;
    if (!r.pod(&v)) return nullptr;
    return std::make_unique<FloatPDLAttr>(tag, v);
  }
  if (tag == "denseElementsAttr") return parseDense(r, tag);
  if (tag == "array") {
    int64_t n = 0;
    if (!r.pod(&n) || n < 0 || n > kMaxCount) return nullptr;
    auto arr = std::make_unique<ArrayPDLAttr>(tag);
    for (int64_t i = 0; i < n; ++i) {
      PDLAttrPtr v = parseAny(r, depth + 1);
      if (!v) return nullptr;
      arr->push_back(std::move(v));
    }
    return arr;
  }
  if (tag == "intArray") {
    int64_t n = 0;
    if (!r.pod(&n) || n < 0 || n > kMaxCount) return nullptr;
    auto arr = std::make_unique<IntArrayPDLAttr>(tag);
    for (int64_t i = 0; i < n; ++i) {
      int64_t v = 0;
      if (!r.pod(&v)) return nullptr;
      arr->push_back(v);
    }
    return arr;
  }
  return nullptr;
}

}  // namespace

std::unique_ptr<PDLAttr> parsePDLAttr(const uint8_t* buffer, size_t size, size_t* consumed) {
  Reader r(buffer, size);
  PDLAttrPtr out = parseAny(r, 0);
  if (consumed) *consumed = out ? static_cast<size_t>(r.pos() - buffer) : 0;
  return out;
}

std::unique_ptr<PDLAttr> parsePDLAttr(uint8_t*& buffer) {
  // The compiled program hands over a bare pointer: the blob's own length fields
  // are the only bound available.
  size_t used = 0;
  PDLAttrPtr out = parsePDLAttr(buffer, std::numeric_limits<size_t>::max() / 2, &used);
  buffer += used;
  return out;
}

}  // namespace ral
}  // namespace tao
