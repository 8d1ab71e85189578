// Vector-ALU tile kernels for element type double: one instantiation per semiring
// the reference pre-tunes (include/cuasr/gemm/device/default_srgemm_configuration.h:44-275);
// min-times and max-times live in strict_valu.hip.
#include "valu_tile.h"

namespace cuasr_amd {

#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return launch_valu_sized<double, ADD, MUL, 8, 4, 16, 4, 4>;

launch_fn find_valu_strict(int dtype, int add_op, int mult_op);

launch_fn find_valu_f64(int add_op, int mult_op) {
  PAIR(kPlus, kMultiplies)
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kMinimum, kMaximum)
  PAIR(kMaximum, kMinimum)
  PAIR(kLogicalOr, kLogicalAnd)
  return find_valu_strict(CUASR_AMD_F64, add_op, mult_op);
}

}  // namespace cuasr_amd
