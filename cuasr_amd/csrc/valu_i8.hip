// The packed half-precision tile (half_tile.h) for operands that are not binary16: int8 (exact in binary16 for the
// tropical pairs), and the 4- and 8-byte types for or-and, whose operands reach LDS as masks.
#include "half_tile.h"

namespace cuasr_amd {

// int8 operands: the pairs whose terms are sums, minima or maxima of two int8 values (exact in binary16), the two
// whose terms are products (exact as 16-bit integers), the bitwise pairs (the same lanes), and or-and
launch_fn find_valu_i8(int add_op, int mult_op) {
#define PAIR(ADD, MUL) \
  if (add_op == ADD && mult_op == MUL) return half_tile::launch<ADD, MUL, int8_t>;
  PAIR(kMinimum, kPlus)
  PAIR(kMaximum, kPlus)
  PAIR(kMinimum, kMaximum)
  PAIR(kMaximum, kMinimum)
  PAIR(kMinimum, kMultiplies)   // (int16 lanes)
  PAIR(kMaximum, kMultiplies)
  PAIR(kBitXor, kBitAnd)
  PAIR(kBitOr, kBitAnd)
  PAIR(kLogicalOr, kLogicalAnd)
#undef PAIR
  return nullptr;
}

// or-and on float / double / 32-bit integer operands.  The operators only ask whether an operand is zero, so nothing
// of the element type survives the trip to LDS: large outputs take the 16-bit mask form of the packed tile (two terms per
// three-input bit operation; 4096^3: 128 TOPS against 84 on the staged tile's 32-bit masks), smaller ones, which the
// packed tile's large workgroups would leave most of the chip idle on, stay on the staged tile.
launch_fn find_valu_f32(int add_op, int mult_op);
launch_fn find_valu_f64(int add_op, int mult_op);
launch_fn find_valu_i32(int add_op, int mult_op);
launch_fn find_valu_u32(int add_op, int mult_op);
template <typename T> static launch_fn staged_or_and() {
  if constexpr (std::is_same<T, float>::value) return find_valu_f32(kLogicalOr, kLogicalAnd);
  else if constexpr (std::is_same<T, double>::value) return find_valu_f64(kLogicalOr, kLogicalAnd);
  else if constexpr (std::is_same<T, int32_t>::value) return find_valu_i32(kLogicalOr, kLogicalAnd);
  else return find_valu_u32(kLogicalOr, kLogicalAnd);
}
template <typename T> static hipError_t or_and_on_masks(const Problem &p, hipStream_t s) {
  const long long full = (long long)((p.m + 127) / 128) * ((p.n + 255) / 256) * (p.workspace ? p.slices : 1) * p.batch;
  // (8-byte operands from 128 such tiles on: their staged tile is slower, 2048^3 58 against 65 - 68 TOPS)
  if (full >= (sizeof(T) == 8 ? 128 : 384)) return half_tile::launch<kLogicalOr, kLogicalAnd, T>(p, s);
  const launch_fn staged = staged_or_and<T>();
  return staged ? staged(p, s) : hipErrorNotSupported;
}
launch_fn find_or_and_on_masks(int dtype) {
  if (dtype == CUASR_AMD_F32) return or_and_on_masks<float>;
  if (dtype == CUASR_AMD_F64) return or_and_on_masks<double>;
  if (dtype == CUASR_AMD_I32) return or_and_on_masks<int32_t>;
  if (dtype == CUASR_AMD_U32) return or_and_on_masks<uint32_t>;
  return nullptr;
}

}  // namespace cuasr_amd
