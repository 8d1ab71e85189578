// Direct-to-LDS vector-ALU tiles, element type double.
#include "direct64_tile.h"

namespace cuasr_amd {

#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return launch_direct64<double, ADD, MUL>;

launch_fn find_direct_f64(int add_op, int mult_op) {
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kPlus, kMultiplies)
  PAIR(kMinimum, kMaximum)
  PAIR(kMaximum, kMinimum)
  return nullptr;
}

bool direct64_can_run(const Problem &p) { return direct64_ok(p); }

}  // namespace cuasr_amd
