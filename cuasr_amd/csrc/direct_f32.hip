// Direct-to-LDS vector-ALU tiles, element type float.
#include "direct_tile.h"

namespace cuasr_amd {

#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return launch_direct<float, ADD, MUL>;

launch_fn find_direct_f32(int add_op, int mult_op) {
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kPlus, kMultiplies)
  PAIR(kMinimum, kMaximum)
  PAIR(kMaximum, kMinimum)
  PAIR(kLogicalOr, kLogicalAnd)
  return nullptr;
}

bool direct_can_run(const Problem &p) { return direct_ok(p); }

}  // namespace cuasr_amd
