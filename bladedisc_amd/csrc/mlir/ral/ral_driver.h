// Base class of a device driver facade owned by a RAL context
// (reference: tao_compiler/mlir/ral/ral_driver.h).
#ifndef RAL_RAL_DRIVER_H_
#define RAL_RAL_DRIVER_H_

#include "mlir/ral/ral_base.h"

namespace tao {
namespace ral {

class Driver {
 public:
  virtual ~Driver() = default;
};

}  // namespace ral
}  // namespace tao

#endif  // RAL_RAL_DRIVER_H_
