// The packed half-precision tile (half_tile.h) for binary16 operands: all eight pre-tuned semirings.
#include "half_tile.h"

namespace cuasr_amd {

// The semirings whose operators are each one packed instruction.  Sums, minima and maxima of data free of -0
// never produce -0; products do, so min-times and max-times settle the sign of a zero result in the epilogue
// (ZERO_SIGN in the kernel).  or-and runs on masks.
launch_fn find_valu_f16(int add_op, int mult_op) {
#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return half_tile::launch<ADD, MUL>;
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kMinimum, kMaximum)
  PAIR(kMaximum, kMinimum)
  PAIR(kPlus, kMultiplies)
  PAIR(kMinimum, kMultiplies)
  PAIR(kMaximum, kMultiplies)
  PAIR(kLogicalOr, kLogicalAnd)
#undef PAIR
  return nullptr;
}

}  // namespace cuasr_amd
