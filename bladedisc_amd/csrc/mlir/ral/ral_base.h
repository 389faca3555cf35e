// Basic vocabulary types of RAL, the runtime abstraction layer that compiled DISC
// programs call into.  Same names and meaning as the reference's
// tao_compiler/mlir/ral/ral_base.h so that kernel sources written against it
// compile unchanged.
#ifndef RAL_RAL_BASE_H_
#define RAL_RAL_BASE_H_

#include <cstddef>
#include <cstdint>
#include <functional>
#include <vector>

namespace tao {
namespace ral {

using status_t = int32_t;          // 0 = ok
using buffer_t = void*;            // device or host memory
using const_buffer_t = const void*;
using opaque_t = void*;            // platform handle (e.g. a hipStream_t)
using buffer_shape_t = std::vector<int64_t>;

// Type-erased entry point: every registered function is called through a
// void** whose slots point at the scalar arguments (and result slots).
using api_func_t = std::function<void(void**)>;

using alloc_t = std::function<buffer_t(size_t)>;
using dealloc_t = std::function<void(buffer_t)>;

struct Allocator {
  virtual ~Allocator() = default;
  virtual void releaseAllFreeBuffers() {}
  virtual buffer_t alloc(size_t bytes) = 0;
  virtual void dealloc(buffer_t buffer) = 0;
};

}  // namespace ral
}  // namespace tao

#endif  // RAL_RAL_BASE_H_
