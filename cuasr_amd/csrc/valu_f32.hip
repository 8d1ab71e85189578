// Vector-ALU tile kernels for element type float: one instantiation per semiring
// the reference pre-tunes (include/cuasr/gemm/device/default_srgemm_configuration.h:44-275);
// min-times and max-times live in strict_valu.hip.
#include "valu_tile.h"

namespace cuasr_amd {

// k-tile 32: one barrier per 32 k costs visibly less than one per 16 (68.9 -> 73.2 TOPS, min-plus 4096^3)
#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return launch_valu_sized<float, ADD, MUL, 8, 8, 32, 4, 4>;

launch_fn find_valu_strict(int dtype, int add_op, int mult_op);

launch_fn find_valu_f32(int add_op, int mult_op) {
  PAIR(kPlus, kMultiplies)
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kMinimum, kMaximum)
  PAIR(kMaximum, kMinimum)
  PAIR(kLogicalOr, kLogicalAnd)
  return find_valu_strict(CUASR_AMD_F32, add_op, mult_op);
}

}  // namespace cuasr_amd
