// Hand-scheduled main loops of the 4-wave direct-to-LDS tile (direct_tile.h) for the semirings whose term
// is a fixed group of vector instructions.  The schedule (order of the groups, LDS reads, waits, the
// barrier, the global -> LDS fetch) comes from gen_direct_asm.py; the arithmetic of a group is given here.
//
//   AsmLoop<T, ADD, MUL, A_KC, B_KC>::type   the loop for that element type, semiring and pair of
//                                            panel forms, or void where there is none
#pragma once
#include "semiring.h"

namespace cuasr_amd {

typedef float asm_v16 __attribute__((ext_vector_type(16)));

// The registers a loop lives in: acc[i / 2][(i % 2) * 8 + j] is accumulator (i, j) and sits in v(8 i + j);
// frag is v64 .. v111, the fragments carried from one k-tile to the next.  Element types other than float
// travel as bit patterns.
struct AsmRegs {
  asm_v16 acc[4];
  asm_v16 frag[3];
};

#define CUASR_MUL2_ADD3(MULOP, ADD3OP, acc, t0, t1, q0, p0, q1, p1)                                           \
  MULOP " " t0 ", " q0 ", " p0 "\n" MULOP " " t1 ", " q1 ", " p1 "\n" ADD3OP " " acc ", " acc ", " t0 ", " t1 "\n"
#define CUASR_BITOP3(TABLE, acc, t0, t1, q0, p0, q1, p1)                                                      \
  "v_bitop3_b32 " acc ", " q0 ", " p0 ", " acc " bitop3:" TABLE "\nv_bitop3_b32 " acc ", " q1 ", " p1 ", " acc " bitop3:" TABLE "\n"

// ---- one struct per (semiring, pair of panel forms)
#define CUASR_ASM_FORMS(NAME)                                 \
  CUASR_ASM_ONE(NAME##_kx, "gen/direct_asm_kx_prime.inc", "gen/direct_asm_kx_tile.inc") \
  CUASR_ASM_ONE(NAME##_xx, "gen/direct_asm_xx_prime.inc", "gen/direct_asm_xx_tile.inc") \
  CUASR_ASM_ONE(NAME##_xk, "gen/direct_asm_xk_prime.inc", "gen/direct_asm_xk_tile.inc")

namespace asm_loops {

#define CUASR_TERM2(acc, t0, t1, q0, p0, q1, p1) CUASR_MUL2_ADD3("v_add_f32", "v_min3_f32", acc, t0, t1, q0, p0, q1, p1)
#define CUASR_ASM_STRUCT min_plus_f32_kx
#define CUASR_ASM_PRIME_INC "gen/direct_asm_kx_prime.inc"
#define CUASR_ASM_TILE_INC "gen/direct_asm_kx_tile.inc"
#include "direct_asm_instance.h"
#undef CUASR_ASM_STRUCT
#undef CUASR_ASM_PRIME_INC
#undef CUASR_ASM_TILE_INC
#undef CUASR_TERM2

}  // namespace asm_loops

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC> struct AsmLoop { typedef void type; };
template <> struct AsmLoop<float, kMinimum, kPlus, true, false> { typedef asm_loops::min_plus_f32_kx type; };

}  // namespace cuasr_amd
