// Direct-to-LDS vector-ALU tiles, element type uint32_t.
#include "direct_tile.h"

namespace cuasr_amd {

#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return launch_direct<uint32_t, ADD, MUL>;

launch_fn find_direct_u32(int add_op, int mult_op) {
  PAIR(kBitXor, kBitAnd)
  PAIR(kBitXor, kLogicalAnd)
  PAIR(kBitOr, kBitAnd)
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kPlus, kMultiplies)
  return nullptr;
}

}  // namespace cuasr_amd
