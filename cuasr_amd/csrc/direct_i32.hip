// Direct-to-LDS vector-ALU tiles, element type int32_t.
#include "direct_tile.h"

namespace cuasr_amd {

#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return launch_direct<int32_t, ADD, MUL>;

launch_fn find_direct_i32(int add_op, int mult_op) {
  PAIR(kBitXor, kBitAnd)
  PAIR(kBitXor, kLogicalAnd)
  PAIR(kBitOr, kBitAnd)
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kPlus, kMultiplies)
  return nullptr;
}

// the semirings whose stream-K form is exact: the add neither depends on the order or grouping of its
// terms nor has to be distributed over (alpha is the multiplicative identity there)
streamk_fn find_streamk_i32(int add_op, int mult_op) {
  if (add_op == kBitXor && mult_op == kBitAnd) return launch_direct_streamk<int32_t, kBitXor, kBitAnd>;
  if (add_op == kBitOr && mult_op == kBitAnd) return launch_direct_streamk<int32_t, kBitOr, kBitAnd>;
  return nullptr;
}

}  // namespace cuasr_amd
