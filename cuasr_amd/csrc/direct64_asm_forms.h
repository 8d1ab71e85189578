// The hand-scheduled main loops of one 8-byte semiring, one per pair of panel forms.  Included once per
// semiring by direct_asm.h, which defines CUASR_ASM_SEMIRING (an identifier) and CUASR_TERM1 (see
// direct64_asm_instance.h).  No include guard on purpose.
#define CUASR_ASM_STRUCT CUASR_ASM_CAT(CUASR_ASM_SEMIRING, _kx)
#define CUASR_ASM_PRIME_INC "gen/direct_asm_d_kx_prime.inc"
#define CUASR_ASM_TILE_INC "gen/direct_asm_d_kx_tile.inc"
#include "direct64_asm_instance.h"
#undef CUASR_ASM_STRUCT
#undef CUASR_ASM_PRIME_INC
#undef CUASR_ASM_TILE_INC

#define CUASR_ASM_STRUCT CUASR_ASM_CAT(CUASR_ASM_SEMIRING, _xx)
#define CUASR_ASM_PRIME_INC "gen/direct_asm_d_xx_prime.inc"
#define CUASR_ASM_TILE_INC "gen/direct_asm_d_xx_tile.inc"
#include "direct64_asm_instance.h"
#undef CUASR_ASM_STRUCT
#undef CUASR_ASM_PRIME_INC
#undef CUASR_ASM_TILE_INC

#define CUASR_ASM_STRUCT CUASR_ASM_CAT(CUASR_ASM_SEMIRING, _xk)
#define CUASR_ASM_PRIME_INC "gen/direct_asm_d_xk_prime.inc"
#define CUASR_ASM_TILE_INC "gen/direct_asm_d_xk_tile.inc"
#include "direct64_asm_instance.h"
#undef CUASR_ASM_STRUCT
#undef CUASR_ASM_PRIME_INC
#undef CUASR_ASM_TILE_INC

#define CUASR_ASM_STRUCT CUASR_ASM_CAT(CUASR_ASM_SEMIRING, _kk)
#define CUASR_ASM_PRIME_INC "gen/direct_asm_d_kk_prime.inc"
#define CUASR_ASM_TILE_INC "gen/direct_asm_d_kk_tile.inc"
#include "direct64_asm_instance.h"
#undef CUASR_ASM_STRUCT
#undef CUASR_ASM_PRIME_INC
#undef CUASR_ASM_TILE_INC
