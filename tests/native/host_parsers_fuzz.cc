// Host-side robustness check of the two parsers that read bytes a compiled program hands to
// the runtime: the custom-call attribute blob (pdll_util) and the constant-store file
// (ral_metadata).  Built with -fsanitize=address,undefined by tests/test_host_sanitized.py.
// A valid input is built, parsed, then truncated at every length and mutated a few thousand
// times with a fixed seed: every outcome must be "parsed" or "rejected" -- never a read
// outside the buffer, an overflow or a crash (the sanitizers abort the process on those).
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <string>
#include <vector>

#include "mlir/ral/context/conv_attr_util.h"
#include "mlir/ral/context/pdll_util.h"
#include "mlir/ral/ral_metadata.h"

using tao::ral::MetadataFile;
using tao::ral::MetadataFileEmitter;

namespace {

struct Blob {
  std::vector<uint8_t> b;
  void i64(int64_t v) { raw(&v, 8); }
  void u32(unsigned v) { raw(&v, sizeof v); }
  void f64(double v) { raw(&v, 8); }
  void byte(uint8_t v) { b.push_back(v); }
  void str(const std::string& s) { i64((int64_t)s.size()); raw(s.data(), s.size()); }
  void raw(const void* p, size_t n) { b.insert(b.end(), (const uint8_t*)p, (const uint8_t*)p + n); }
};

Blob sample_attrs() {
  Blob x;
  x.str("dict");
  x.i64(7);
  x.str("data_format"); x.str("str"); x.str("NHWC");
  x.str("transpose_b"); x.str("bool"); x.byte(1);
  x.str("axis"); x.str("int"); x.i64(3);
  x.str("eps"); x.str("float"); x.f64(1e-5);
  x.str("strides"); x.str("intArray"); x.i64(4); for (int i = 0; i < 4; ++i) x.i64(1 + i % 2);
  x.str("nested"); x.str("array"); x.i64(2);
  x.str("str"); x.str("SAME");
  x.str("intArray"); x.i64(2); x.i64(5); x.i64(6);
  x.str("dense"); x.str("denseElementsAttr"); x.str("int"); x.u32(32); x.i64(2); x.i64(2); x.i64(3);
  x.byte(0);
  std::string rawdata(24, '\x01');
  x.str(rawdata);
  return x;
}

unsigned rng_state = 12345;
unsigned rnd() { rng_state = rng_state * 1664525u + 1013904223u; return rng_state >> 8; }

int fuzz_attrs() {
  const Blob good = sample_attrs();
  size_t used = 0;
  auto attr = tao::ral::parsePDLAttr(good.b.data(), good.b.size(), &used);
  if (!attr || used != good.b.size() || attr->getType() != "dict") {
    std::printf("attrs: the valid blob was not parsed (used %zu of %zu)\n", used, good.b.size());
    return 1;
  }
  auto& dict = attr->as<tao::ral::DictPDLAttr>();
  if (!dict.hasKey("dense") || dict.get("axis").as<tao::ral::IntPDLAttr>().getValue() != 3) return 1;
  int parsed = 0, rejected = 0;
  for (size_t n = 0; n < good.b.size(); ++n) {           // every truncation, on an exact-size copy
    std::vector<uint8_t> cut(good.b.begin(), good.b.begin() + n);
    (tao::ral::parsePDLAttr(cut.data(), cut.size(), &used) ? parsed : rejected)++;
  }
  if (parsed != 0) { std::printf("attrs: a truncated blob was accepted\n"); return 1; }
  for (int it = 0; it < 20000; ++it) {                    // byte and length mutations
    std::vector<uint8_t> m = good.b;
    const int edits = 1 + rnd() % 4;
    for (int e = 0; e < edits; ++e) {
      const size_t at = rnd() % m.size();
      switch (rnd() % 4) {
        case 0: m[at] = (uint8_t)rnd(); break;
        case 1: m[at] = 0xff; break;
        case 2: if (at + 8 <= m.size()) { int64_t v = (int64_t)1 << (rnd() % 63); std::memcpy(&m[at], &v, 8); } break;
        default: if (at + 8 <= m.size()) { int64_t v = -(int64_t)(rnd() % 1000); std::memcpy(&m[at], &v, 8); } break;
      }
    }
    (tao::ral::parsePDLAttr(m.data(), m.size(), &used) ? parsed : rejected)++;
  }
  std::printf("attrs: %d mutated blobs parsed, %d rejected\n", parsed, rejected);
  return 0;
}

int fuzz_metadata(const std::string& dir) {
  const std::string path = dir + "/consts.metadata";
  {
    MetadataFileEmitter em(path);
    if (!em.emitHeader()) return 1;
    if (!em.emitHostConstant("0_i32_4", "0100000002000000")) return 1;
    if (!em.emitDeviceConstant("1_i8_2x3", "010203040506")) return 1;
    if (em.emitDeviceConstant("1_i8_2x3", "00")) { std::printf("metadata: duplicate accepted\n"); return 1; }
    if (!em.emitTailer()) return 1;
  }
  std::ifstream in(path, std::ios::binary);
  std::vector<char> good((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
  auto file = MetadataFile::loadFromFile(path);
  const std::string* data = nullptr;
  if (!file || !file->getDeviceConstant("1_i8_2x3", data) || *data != "010203040506") {
    std::printf("metadata: the valid file was not read back\n");
    return 1;
  }
  const std::string mpath = dir + "/mutated.metadata";
  auto write = [&](const std::vector<char>& v) {
    std::ofstream out(mpath, std::ios::binary | std::ios::trunc);
    out.write(v.data(), (std::streamsize)v.size());
  };
  int loaded = 0, rejected = 0;
  for (size_t n = 0; n < good.size(); ++n) {
    write(std::vector<char>(good.begin(), good.begin() + n));
    (MetadataFile::loadFromFile(mpath) ? loaded : rejected)++;
  }
  if (loaded != 0) { std::printf("metadata: a truncated file was accepted\n"); return 1; }
  for (int it = 0; it < 3000; ++it) {
    std::vector<char> m = good;
    const size_t at = rnd() % m.size();
    if (rnd() % 2 && at + 8 <= m.size()) {
      uint64_t v = (uint64_t)1 << (rnd() % 64);
      std::memcpy(&m[at], &v, 8);
    } else {
      m[at] = (char)rnd();
    }
    write(m);
    (MetadataFile::loadFromFile(mpath) ? loaded : rejected)++;
  }
  std::printf("metadata: %d mutated files loaded, %d rejected\n", loaded, rejected);
  return 0;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 2) { std::printf("usage: %s <scratch dir>\n", argv[0]); return 2; }
  if (fuzz_attrs()) return 1;
  if (fuzz_metadata(argv[1])) return 1;
  std::printf("ok\n");
  return 0;
}
