// One hand-scheduled main loop of the 4-wave direct-to-LDS tile for 8-byte element types: the generated
// schedule of one pair of panel forms (gen/direct_asm_d_<form>_{prime,tile}.inc, written by
// gen_direct_asm.py) with the arithmetic of one semiring.  Included once per (form, semiring) by
// direct_asm.h, which defines CUASR_ASM_STRUCT, CUASR_ASM_PRIME_INC, CUASR_ASM_TILE_INC and
//   CUASR_TERM1(acc, t, q, p)   asm text of acc <- add(acc, mult(q, p)) on register pairs
// No include guard on purpose.
struct CUASR_ASM_STRUCT {
  // fragments of the first k-pair into their registers; the tile must have landed in LDS stage 0
  static __device__ __forceinline__ void prime(AsmRegs &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include CUASR_ASM_PRIME_INC
        : "+{v[64:79]}"(r.frag[0]), "+{v[80:95]}"(r.frag[1]), "+{v[96:111]}"(r.frag[2])
        : [a_addr] "v"(a_addr), [b_addr] "v"(b_addr)
        : "memory");
  }
  // one k-tile of 16: 512 terms per lane, the workgroup barrier that hands the LDS stage back, the fetch of
  // the tile two ahead into it (if fetch > 0), and the fragments of the next tile's first k-pair
  static __device__ __forceinline__ void tile(AsmRegs &r, unsigned &a_addr, unsigned &b_addr, unsigned a_step, unsigned b_step,
                                              int fetch, unsigned m0_a, unsigned m0_b, unsigned off_a0, unsigned off_a1,
                                              unsigned off_b0, unsigned off_b1, const char *base_a, const char *base_b) {
    unsigned m0_save;
    asm volatile(
#include CUASR_ASM_TILE_INC
        : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]),
          "+{v[64:79]}"(r.frag[0]), "+{v[80:95]}"(r.frag[1]), "+{v[96:111]}"(r.frag[2]),
          [a_addr] "+v"(a_addr), [b_addr] "+v"(b_addr), [m0_save] "=&s"(m0_save)
        : [a_step] "s"(a_step), [b_step] "s"(b_step), [fetch] "s"(fetch), [m0_a] "s"(m0_a), [m0_b] "s"(m0_b),
          [off_a0] "v"(off_a0), [off_a1] "v"(off_a1), [off_b0] "v"(off_b0), [off_b1] "v"(off_b1),
          [base_a] "s"(base_a), [base_b] "s"(base_b)
        : "v112", "v113", "v114", "v115", "scc", "memory");
  }
};
