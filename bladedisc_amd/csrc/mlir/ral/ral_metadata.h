// The constant store that accompanies a compiled program: large constants are not
// linked into the program but written to a side file at compile time and fetched by
// name at run time (ral_const).  File layout, as the reference's compiler emits it
// (tao_compiler/mlir/ral/ral_metadata.cc:60-200), host byte order:
//   u64   magic 0x1234567890ABCDEF
//   n x { u8 is_host; u64 key_len; key; u64 value_len; value }
//   u64   n
// A value is the constant's bytes as a hexadecimal string.
#ifndef RAL_RAL_METADATA_H_
#define RAL_RAL_METADATA_H_

#include <cstdint>
#include <fstream>
#include <memory>
#include <string>
#include <unordered_map>

namespace tao {
namespace ral {

class MetadataFile {
 public:
  // nullptr when the file is missing, truncated or does not start with the magic
  static std::unique_ptr<MetadataFile> loadFromFile(const std::string& filename);

  bool getHostConstant(const std::string& name, const std::string*& data);
  bool releaseHostConstant(const std::string& name);
  bool getDeviceConstant(const std::string& name, const std::string*& data);
  bool releaseDeviceConstant(const std::string& name);

 private:
  MetadataFile() = default;
  MetadataFile(const MetadataFile&) = delete;
  MetadataFile& operator=(const MetadataFile&) = delete;

  std::unordered_map<std::string, std::string> host_;
  std::unordered_map<std::string, std::string> device_;
};

// Writes a metadata file: emitHeader, any number of emit*Constant, emitTailer.
class MetadataFileEmitter {
 public:
  explicit MetadataFileEmitter(const std::string& filename) : filename_(filename) {}
  MetadataFileEmitter(const MetadataFileEmitter&) = delete;
  MetadataFileEmitter& operator=(const MetadataFileEmitter&) = delete;

  bool emitHeader();
  // false on a duplicated name or an I/O error
  bool emitHostConstant(const std::string& name, const std::string& data);
  bool emitDeviceConstant(const std::string& name, const std::string& data);
  bool emitTailer();
  int getNumHostConstantEmitted() const { return num_host_; }
  int getNumDeviceConstantEmitted() const { return num_device_; }

 private:
  bool emitRecord(bool is_host, const std::string& name, const std::string& data);

  std::string filename_;
  std::ofstream out_;
  std::unordered_map<std::string, bool> seen_;  // name -> is_host
  int num_host_ = 0;
  int num_device_ = 0;
};

}  // namespace ral
}  // namespace tao

#endif  // RAL_RAL_METADATA_H_
