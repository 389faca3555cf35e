#include "mlir/ral/ral_metadata.h"

#include <vector>

namespace tao {
namespace ral {

namespace {

constexpr uint64_t kMagic = 0x1234567890ABCDEFull;
// a constant larger than this is a corrupt length field, not a constant
constexpr uint64_t kMaxField = 1ull << 40;

bool readU64(std::ifstream& in, uint64_t* v) {
  in.read(reinterpret_cast<char*>(v), sizeof(*v));
  return static_cast<bool>(in);
}

bool readString(std::ifstream& in, uint64_t remaining, std::string* s) {
  uint64_t len = 0;
  if (!readU64(in, &len) || len > kMaxField || len > remaining) return false;
  s->assign(len, '\0');
  if (len) in.read(&(*s)[0], (std::streamsize)len);
  return static_cast<bool>(in);
}

bool writeU64(std::ofstream& out, uint64_t v) {
  out.write(reinterpret_cast<const char*>(&v), sizeof(v));
  return static_cast<bool>(out);
}

bool writeString(std::ofstream& out, const std::string& s) {
  if (!writeU64(out, s.size())) return false;
  out.write(s.data(), (std::streamsize)s.size());
  return static_cast<bool>(out);
}

}  // namespace

std::unique_ptr<MetadataFile> MetadataFile::loadFromFile(const std::string& filename) {
  std::ifstream in(filename, std::ios::in | std::ios::binary);
  if (!in) return nullptr;
  in.seekg(0, std::ios::end);
  const uint64_t size = (uint64_t)in.tellg();
  if (size < 2 * sizeof(uint64_t)) return nullptr;
  in.seekg(0);
  uint64_t magic = 0;
  if (!readU64(in, &magic) || magic != kMagic) return nullptr;
  in.seekg(-(std::streamoff)sizeof(uint64_t), std::ios::end);
  uint64_t count = 0;
  if (!readU64(in, &count) || count > size) return nullptr;
  in.seekg(sizeof(uint64_t));
  std::unique_ptr<MetadataFile> file(new MetadataFile);
  for (uint64_t i = 0; i < count; ++i) {
    char is_host = 0;
    in.read(&is_host, 1);
    if (!in) return nullptr;
    std::string key, value;
    if (!readString(in, size, &key) || !readString(in, size, &value)) return nullptr;
    (is_host ? file->host_ : file->device_).emplace(std::move(key), std::move(value));
  }
  return file;
}

bool MetadataFile::getHostConstant(const std::string& name, const std::string*& data) {
  auto it = host_.find(name);
  if (it == host_.end()) return false;
  data = &it->second;
  return true;
}

bool MetadataFile::releaseHostConstant(const std::string& name) { return host_.erase(name) != 0; }

bool MetadataFile::getDeviceConstant(const std::string& name, const std::string*& data) {
  auto it = device_.find(name);
  if (it == device_.end()) return false;
  data = &it->second;
  return true;
}

bool MetadataFile::releaseDeviceConstant(const std::string& name) {
  return device_.erase(name) != 0;
}

bool MetadataFileEmitter::emitHeader() {
  out_.open(filename_, std::ios::out | std::ios::binary | std::ios::trunc);
  return out_ && writeU64(out_, kMagic);
}

bool MetadataFileEmitter::emitRecord(bool is_host, const std::string& name,
                                     const std::string& data) {
  // host and device constants live in separate name spaces
  const std::string scoped = (is_host ? "h:" : "d:") + name;
  if (!out_ || !seen_.emplace(scoped, is_host).second) return false;
  const char flag = is_host ? 1 : 0;
  out_.write(&flag, 1);
  if (!out_ || !writeString(out_, name) || !writeString(out_, data)) return false;
  ++(is_host ? num_host_ : num_device_);
  return true;
}

bool MetadataFileEmitter::emitHostConstant(const std::string& name, const std::string& data) {
  return emitRecord(true, name, data);
}

bool MetadataFileEmitter::emitDeviceConstant(const std::string& name, const std::string& data) {
  return emitRecord(false, name, data);
}

bool MetadataFileEmitter::emitTailer() {
  if (!out_ || !writeU64(out_, (uint64_t)(num_host_ + num_device_))) return false;
  out_.close();
  return true;
}

}  // namespace ral
}  // namespace tao
