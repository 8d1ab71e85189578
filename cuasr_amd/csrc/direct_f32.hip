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

// the semirings whose stream-K form is exact: the add neither depends on the order or grouping of its
// terms nor has to be distributed over (alpha is the multiplicative identity there)
streamk_fn find_streamk_f32(int add_op, int mult_op) {
  if (add_op == kMinimum && mult_op == kPlus) return launch_direct_streamk<float, kMinimum, kPlus>;
  if (add_op == kMaximum && mult_op == kPlus) return launch_direct_streamk<float, kMaximum, kPlus>;
  if (add_op == kMaximum && mult_op == kMinimum) return launch_direct_streamk<float, kMaximum, kMinimum>;
  if (add_op == kMinimum && mult_op == kMaximum) return launch_direct_streamk<float, kMinimum, kMaximum>;
  return nullptr;
}

}  // namespace cuasr_amd
