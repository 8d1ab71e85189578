// Hand-scheduled main loops of the 4-wave direct-to-LDS tile (direct_tile.h) for the semirings whose term
// is a fixed group of vector instructions.  The schedule (order of the groups, LDS reads, waits, the
// barrier, the global -> LDS fetch) comes from gen_direct_asm.py; the arithmetic of a group is given here.
//
//   AsmLoop<T, ADD, MUL, A_KC, B_KC>::type   the loop for that element type, semiring and pair of
//                                            panel forms, or void where there is none
//
// The operators are those of semiring.h: floating-point minimum / maximum are the hardware instructions
// (the data is free of NaN and of -0, the same contract as the compiled tiles), sums and products are
// single rounded operations (no fused multiply-add), and plus-times adds its products in ascending k.
#pragma once
#include "semiring.h"

namespace cuasr_amd {

typedef float asm_v16 __attribute__((ext_vector_type(16)));

// The registers a loop lives in.  4-byte types: acc[i / 2][(i % 2) * 8 + j] is accumulator (i, j) of the 8 x 8
// tile and sits in v(8 i + j); 8-byte types: accumulator (i, j) of the 8 x 4 tile is the register pair
// v[8 i + 2 j : 8 i + 2 j + 1], low word first, i.e. elements (i % 2) * 8 + 2 j and + 1 of acc[i / 2].
// frag is v64 .. v111, the fragments carried from one k-tile to the next.  Everything travels as bit patterns.
struct AsmRegs {
  asm_v16 acc[4];
  asm_v16 frag[3];
};

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC> struct AsmLoop { typedef void type; };

#define CUASR_ASM_CAT_(a, b) a##b
#define CUASR_ASM_CAT(a, b) CUASR_ASM_CAT_(a, b)
// acc <- ADD3(acc, MUL(q0, p0), MUL(q1, p1)): two products and one three-input fold
#define CUASR_MUL2_FOLD3(MULOP, ADD3OP, acc, t0, t1, q0, p0, q1, p1) \
  MULOP " " t0 ", " q0 ", " p0 "\n" MULOP " " t1 ", " q1 ", " p1 "\n" ADD3OP " " acc ", " acc ", " t0 ", " t1 "\n"
// acc <- (acc + q0 * p0) + q1 * p1, every operation rounded on its own, ascending k
#define CUASR_MUL2_ADD2(MULOP, ADDOP, acc, t0, t1, q0, p0, q1, p1) \
  MULOP " " t0 ", " q0 ", " p0 "\n" MULOP " " t1 ", " q1 ", " p1 "\n" ADDOP " " acc ", " t0 ", " acc "\n" ADDOP " " acc ", " t1 ", " acc "\n"
// acc <- f(q, p, acc) twice, f a three-input bit function given by its truth table
#define CUASR_BITOP3(TABLE, acc, t0, t1, q0, p0, q1, p1) \
  "v_bitop3_b32 " acc ", " q0 ", " p0 ", " acc " bitop3:" TABLE "\nv_bitop3_b32 " acc ", " q1 ", " p1 ", " acc " bitop3:" TABLE "\n"
#define CUASR_ASM_SELECT(T, ADD, MUL, NAME)                                                            \
  template <> struct AsmLoop<T, ADD, MUL, true, false> { typedef asm_loops::NAME##_kx type; };        \
  template <> struct AsmLoop<T, ADD, MUL, false, false> { typedef asm_loops::NAME##_xx type; };       \
  template <> struct AsmLoop<T, ADD, MUL, false, true> { typedef asm_loops::NAME##_xk type; };

namespace asm_loops {

#define CUASR_ASM_SEMIRING min_plus_f32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_add_f32", "v_min3_f32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING max_plus_f32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_add_f32", "v_max3_f32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING max_min_f32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_min_f32", "v_max3_f32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING min_max_f32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_max_f32", "v_min3_f32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING plus_times_f32
#define CUASR_TERM2(...) CUASR_MUL2_ADD2("v_mul_f32", "v_add_f32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING min_plus_i32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_add_u32", "v_min3_i32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING max_plus_i32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_add_u32", "v_max3_i32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING min_plus_u32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_add_u32", "v_min3_u32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING max_plus_u32
#define CUASR_TERM2(...) CUASR_MUL2_FOLD3("v_add_u32", "v_max3_u32", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING xor_and_b32   // acc ^ (q & p): table = value on q = 0xF0, p = 0xCC, acc = 0xAA
#define CUASR_TERM2(...) CUASR_BITOP3("0x6a", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

#define CUASR_ASM_SEMIRING or_and_b32    // acc | (q & p)
#define CUASR_TERM2(...) CUASR_BITOP3("0xea", __VA_ARGS__)
#include "direct_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM2

// ---- 8-byte element types: one term at a time on register pairs (there is no three-input fp64 min / max)
// acc <- ADD(acc, MUL(q, p))
#define CUASR_MUL_FOLD(MULOP, ADDOP, acc, t, q, p) MULOP " " t ", " q ", " p "\n" ADDOP " " acc ", " acc ", " t "\n"
// acc <- q * p + acc with both operations rounded, the product as the left operand like the host reference
#define CUASR_MUL_ADD(MULOP, ADDOP, acc, t, q, p) MULOP " " t ", " q ", " p "\n" ADDOP " " acc ", " t ", " acc "\n"

#define CUASR_ASM_SEMIRING min_plus_f64
#define CUASR_TERM1(...) CUASR_MUL_FOLD("v_add_f64", "v_min_f64", __VA_ARGS__)
#include "direct64_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM1

#define CUASR_ASM_SEMIRING max_plus_f64
#define CUASR_TERM1(...) CUASR_MUL_FOLD("v_add_f64", "v_max_f64", __VA_ARGS__)
#include "direct64_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM1

#define CUASR_ASM_SEMIRING max_min_f64
#define CUASR_TERM1(...) CUASR_MUL_FOLD("v_min_f64", "v_max_f64", __VA_ARGS__)
#include "direct64_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM1

#define CUASR_ASM_SEMIRING min_max_f64
#define CUASR_TERM1(...) CUASR_MUL_FOLD("v_max_f64", "v_min_f64", __VA_ARGS__)
#include "direct64_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM1

#define CUASR_ASM_SEMIRING plus_times_f64
#define CUASR_TERM1(...) CUASR_MUL_ADD("v_mul_f64", "v_add_f64", __VA_ARGS__)
#include "direct64_asm_forms.h"
#undef CUASR_ASM_SEMIRING
#undef CUASR_TERM1

}  // namespace asm_loops

#define CUASR_ASM_SELECT64(ADD, MUL, NAME)                                                                \
  template <> struct AsmLoop<double, ADD, MUL, true, false> { typedef asm_loops::NAME##_kx type; };      \
  template <> struct AsmLoop<double, ADD, MUL, false, false> { typedef asm_loops::NAME##_xx type; };     \
  template <> struct AsmLoop<double, ADD, MUL, false, true> { typedef asm_loops::NAME##_xk type; };      \
  template <> struct AsmLoop<double, ADD, MUL, true, true> { typedef asm_loops::NAME##_kk type; };
CUASR_ASM_SELECT64(kMinimum, kPlus, min_plus_f64)
CUASR_ASM_SELECT64(kMaximum, kPlus, max_plus_f64)
CUASR_ASM_SELECT64(kMaximum, kMinimum, max_min_f64)
CUASR_ASM_SELECT64(kMinimum, kMaximum, min_max_f64)
CUASR_ASM_SELECT64(kPlus, kMultiplies, plus_times_f64)

CUASR_ASM_SELECT(float, kMinimum, kPlus, min_plus_f32)
CUASR_ASM_SELECT(float, kMaximum, kPlus, max_plus_f32)
CUASR_ASM_SELECT(float, kMaximum, kMinimum, max_min_f32)
CUASR_ASM_SELECT(float, kMinimum, kMaximum, min_max_f32)
CUASR_ASM_SELECT(float, kPlus, kMultiplies, plus_times_f32)
CUASR_ASM_SELECT(int32_t, kMinimum, kPlus, min_plus_i32)
CUASR_ASM_SELECT(int32_t, kMaximum, kPlus, max_plus_i32)
CUASR_ASM_SELECT(uint32_t, kMinimum, kPlus, min_plus_u32)
CUASR_ASM_SELECT(uint32_t, kMaximum, kPlus, max_plus_u32)
CUASR_ASM_SELECT(int32_t, kBitXor, kBitAnd, xor_and_b32)
CUASR_ASM_SELECT(uint32_t, kBitXor, kBitAnd, xor_and_b32)
CUASR_ASM_SELECT(int32_t, kBitOr, kBitAnd, or_and_b32)
CUASR_ASM_SELECT(uint32_t, kBitOr, kBitAnd, or_and_b32)

}  // namespace cuasr_amd
