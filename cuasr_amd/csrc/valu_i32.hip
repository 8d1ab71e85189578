// Vector-ALU tile kernels for element type int32_t: one instantiation per semiring
// the reference pre-tunes (include/cuasr/gemm/device/default_srgemm_configuration.h:44-275)
// and, for integers, the GF(2)-style bitwise pairs of
// examples/01_userdefined_semiring/userdefined_semiring.cu:56-99.
#include "valu_tile.h"

namespace cuasr_amd {

#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return launch_valu_sized<int32_t, ADD, MUL, 8, 8, 16, 4, 4>;

launch_fn find_valu_i32(int add_op, int mult_op) {
  PAIR(kPlus, kMultiplies)
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kMinimum, kMultiplies)
  PAIR(kMaximum, kMultiplies)
  PAIR(kMinimum, kMaximum)
  PAIR(kMaximum, kMinimum)
  PAIR(kLogicalOr, kLogicalAnd)
#if 1
  PAIR(kBitXor, kBitAnd)
  PAIR(kBitXor, kLogicalAnd)
  PAIR(kBitOr, kBitAnd)
#endif
  return nullptr;
}

}  // namespace cuasr_amd
