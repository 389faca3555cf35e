// Small memref helpers shared by the kernel entries (reference:
// tao_compiler/mlir/ral/context/context_util.h:47-109).
#ifndef RAL_CONTEXT_CONTEXT_UTIL_H_
#define RAL_CONTEXT_CONTEXT_UTIL_H_

#include <cstdint>

#include "mlir/ral/ral_helper.h"

namespace tao {
namespace ral {

// Dense row-major memref over `ptr` with the given sizes.
template <typename T, int N, typename ShapeTy>
MemRefType<T, N> assignMemRef(void* ptr, const ShapeTy& shape) {
  MemRefType<T, N> m;
  m.basePtr = m.data = static_cast<T*>(ptr);
  m.offset = 0;
  int64_t stride = 1;
  for (int i = N - 1; i >= 0; --i) {
    m.sizes[i] = shape[i];
    m.strides[i] = stride;
    stride *= shape[i];
  }
  return m;
}

template <typename T>
MemRefType<T, 0> assignMemRef_0d(void* ptr) {
  MemRefType<T, 0> m;
  m.basePtr = m.data = static_cast<T*>(ptr);
  m.offset = 0;
  return m;
}

template <typename T, int N>
bool isEmptyMemref(const MemRefType<T, N>& m) {
  for (int i = 0; i < N; ++i)
    if (m.sizes[i] == 0) return true;
  return false;
}

template <typename T>
bool isEmptyMemref(const MemRefType<T, 0>&) {
  return false;
}

template <typename T, int N>
int64_t Size(const MemRefType<T, N>& m) {
  int64_t n = 1;
  for (int i = 0; i < N; ++i) n *= m.sizes[i];
  return n;
}

template <typename T>
int64_t Size(const MemRefType<T, 0>&) {
  return 1;
}

// True when the memref is dense row-major (what the kernels here require).
template <typename T, int N>
bool isContiguous(const MemRefType<T, N>& m) {
  int64_t stride = 1;
  for (int i = N - 1; i >= 0; --i) {
    if (m.sizes[i] != 1 && m.strides[i] != stride) return false;
    stride *= m.sizes[i];
  }
  return true;
}

}  // namespace ral
}  // namespace tao

#endif  // RAL_CONTEXT_CONTEXT_UTIL_H_
