// plus-times on the matrix cores for the narrow element types, hand-scheduled:
//     int8 operands, int32 accumulation and results          v_mfma_i32_32x32x32_i8    (mfma_narrow_kernel, mfma_narrow_kernel_lines)
//     binary16 operands and results, float accumulation      v_mfma_f32_16x16x32_f16   (mfma_narrow_kernel16, mfma_narrow_kernel16_lines)
// for products whose operands are both k-contiguous (A row-major, B column-major in the canonical orientation),
// whose extents are whole tiles of 256 x 256 and whose k range is a multiple of 64 bytes; everything else stays on
// the compiled kernels (mfma_i8.hip, mfma_f16.hip), which take every extent, layout and alignment.  The element
// types are those of the reference's dp4a threadblock cores (include/cuasr/gemm/threadblock/
// default_srmma_core_simt.h:733-1381: int8 operands, never instantiated there) and of its ElementAccumulator =
// float for half operands; the kernel's place is the reference's include/cuasr/gemm/kernel/srgemm.h:156-321.
//
// Either instruction takes 16 consecutive bytes of one row (column) from every lane, and the two kernels share
// tile, ring and loads; each element type has the instruction shape that delivers more of it per watt (loops of
// the bare instructions on random register contents, all at the board's power cap: int8 3.26 POP/s through
// 32 x 32 x 32 against 2.99 through 16 x 16 x 64; binary16 2.07 PFLOP/s through 16 x 16 x 32 against 1.68 through
// 32 x 32 x 16).  The compiled kernels run the matrix cores 24 - 30 % busy: a 64 x 64 wave tile reads 4 KiB of
// fragments per 128 cycles of matrix work, which is all a compute unit's LDS delivers, panels pass through
// registers, and every k-tile ends in a barrier that nothing hides.  Here (the int8 kernel; what differs for
// binary16 is said at its kernel):
//   - workgroup 256 threads = 2 x 2 waves, ONE wave per SIMD; output tile 256 x 256, wave tile 128 x 128 = 4 x 4
//     blocks of 32 x 32: 8 fragment reads per 16 matrix instructions (half the LDS traffic per instruction), and
//     64 KiB of panels per 2^24 operations (half the traffic from L2).  The 256 accumulator registers are the
//     wave's AGPRs; fragments, addresses and the rest live in VGPRs;
//   - panels go global -> LDS without passing registers (global_load_lds_dwordx4).  A stage of the LDS ring is 64
//     bytes of k of both panels; four neighbouring lanes of a load fetch the four 16-byte chunks of one row's 64
//     bytes, so an instruction touches 16 cache lines (one row per lane, 64 lines per instruction, ran into the
//     rate at which a compute unit's L1 looks lines up: 1.2 POP/s, no better than the compiled kernel), and the
//     chunks of a row are stored in an order that depends on the row -- slot 4 r + (c ^ ((r >> 2) & 3)) -- so
//     that a fragment read (32 consecutive rows, one chunk) is free of bank conflicts.  Four stages of 32 KiB;
//   - the main loop is one generated asm statement per stage (gen_direct_asm.py, NarrowMfmaBody): 32 matrix
//     instructions, the 16 fragment reads of the next two steps and the 8 loads of the stage three ahead spread
//     between them, one counted wait and one barrier in the middle of the stage.
// Integer sums wrap modulo 2^32 in any order, so the int8 result is bit-identical to the k-ascending reference
// loop; the binary16 result is the float sum of exact products, rounded to binary16 once (see mfma_f16.hip).
#include "mfma_common.h"

namespace cuasr_amd {
namespace mfma_narrow {

using mfma_panel::tile_coords;

constexpr int BM = 256, BN = 256, STAGE_K_BYTES = 64, STAGES = 4;
constexpr unsigned PANEL = STAGE_K_BYTES * 256;   // bytes of one panel in one stage: 16 KiB

struct Smem {
  unsigned char a[STAGES][PANEL];
  unsigned char b[STAGES][PANEL];
};

typedef int asm_v32 __attribute__((ext_vector_type(32)));
struct Regs {
  asm_v32 acc[8];    // a0 .. a255: block (bm, bn) in a[16 (4 bm + bn) : +15]
  asm_v32 frag[2];   // v0 .. v63: the two fragment buffers
};

__device__ __forceinline__ void dma16(const char *src, unsigned char *lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                   (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
}

#define CUASR_NARROW_ACC                                                                                                  \
  "+{a[0:31]}"(r.acc[0]), "+{a[32:63]}"(r.acc[1]), "+{a[64:95]}"(r.acc[2]), "+{a[96:127]}"(r.acc[3]),                      \
      "+{a[128:159]}"(r.acc[4]), "+{a[160:191]}"(r.acc[5]), "+{a[192:223]}"(r.acc[6]), "+{a[224:255]}"(r.acc[7])
#define CUASR_NARROW_PRIME                                                                                                \
  : "+{v[0:31]}"(r.frag[0]), "+{v[32:63]}"(r.frag[1]) : [a_addr0] "v"(a_addr[0]), [b_addr0] "v"(b_addr[0]) : "memory"
#define CUASR_NARROW_TILE                                                                                                 \
  : CUASR_NARROW_ACC, "+{v[0:31]}"(r.frag[0]), "+{v[32:63]}"(r.frag[1]), [a_addr0] "+v"(a_addr[0]),                       \
    [a_addr1] "+v"(a_addr[1]), [b_addr0] "+v"(b_addr[0]), [b_addr1] "+v"(b_addr[1]), [m0_save] "=&s"(m0_save)             \
  : [step] "s"(step), [fetch] "s"(fetch), [m0_a] "s"(m0_a), [m0_b] "s"(m0_b),                                             \
    [off_a0] "v"(off_a[0]), [off_a1] "v"(off_a[1]), [off_a2] "v"(off_a[2]), [off_a3] "v"(off_a[3]),                       \
    [off_b0] "v"(off_b[0]), [off_b1] "v"(off_b[1]), [off_b2] "v"(off_b[2]), [off_b3] "v"(off_b[3]),                       \
    [base_a] "s"(base_a), [base_b] "s"(base_b)                                                                            \
  : "scc", "memory"
#define CUASR_NARROW_TILE_ARGS                                                                                            \
  Regs &r, unsigned (&a_addr)[2], unsigned (&b_addr)[2], unsigned step, int fetch, unsigned m0_a, unsigned m0_b,          \
      const unsigned (&off_a)[4], const unsigned (&off_b)[4], const char *base_a, const char *base_b

// prime: the fragments of the first step into buffer 0; the stage must have landed in ring slot 0.
// tile: one stage -- 32 matrix instructions per wave, the loads of the stage three ahead (if fetch > 0), the
// workgroup barrier that hands a ring slot back, and the fragments of the next stage's first step.
struct Loop {
  static __device__ __forceinline__ void prime(Regs &r, const unsigned (&a_addr)[2], const unsigned (&b_addr)[2]) {
    asm volatile(
#include "gen/mfma_asm_n_i8_prime.inc"
        CUASR_NARROW_PRIME);
  }
  static __device__ __forceinline__ void tile(CUASR_NARROW_TILE_ARGS) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_n_i8_tile.inc"
        CUASR_NARROW_TILE);
  }
};

// int8 operands, int32 results
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mfma_narrow_kernel(Problem p) {
  using Operand = int8_t;
  using Result = int32_t;
  constexpr long long E = sizeof(Operand);
  __shared__ __attribute__((aligned(1024))) Smem sm;
  select_batch<Result, Operand>(p);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, half = lane >> 5, l32 = lane & 31;
  const int tiles_m = p.m / BM, tiles_n = p.n / BN;   // the host sends whole tiles only
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;

  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const int nstages = (int)((long long)max(ke - kb, 0) * E / STAGE_K_BYTES);   // (the host sends whole stages only)

  Regs r;
#pragma unroll
  for (int v = 0; v < 8; ++v) r.acc[v] = asm_v32(0);
#pragma unroll
  for (int v = 0; v < 2; ++v) r.frag[v] = asm_v32(0);

  if (nstages > 0) {
    const char *base_a = reinterpret_cast<const char *>(p.A) + ((long long)m0 * p.sa_m + kb) * E;
    const char *base_b = reinterpret_cast<const char *>(p.B) + ((long long)n0 * p.sb_n + kb) * E;
    // this wave's 64 rows of each panel in four loads of 16 rows x 64 bytes: lane l of load h fetches row
    // 64 wave + 16 h + l / 4, chunk (l % 4) ^ ((l / 16) % 4) -- the chunk that belongs in the LDS slot the lane writes
    unsigned off_a[4], off_b[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const long long row = wave * 64 + 16 * h + lane / 4;
      const unsigned chunk = (unsigned)((lane & 3) ^ ((lane >> 4) & 3));
      off_a[h] = (unsigned)(row * p.sa_m * E) + 16u * chunk;
      off_b[h] = (unsigned)(row * p.sb_n * E) + 16u * chunk;
    }
    auto fetch = [&](int stage) {
#pragma unroll
      for (int h = 0; h < 4; ++h) dma16(base_a + off_a[h], &sm.a[stage][(wave * 4 + h) * 1024]);
#pragma unroll
      for (int h = 0; h < 4; ++h) dma16(base_b + off_b[h], &sm.b[stage][(wave * 4 + h) * 1024]);
    };
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      if (s < nstages) fetch(s);
      base_a += STAGE_K_BYTES;
      base_b += STAGE_K_BYTES;
    }
    __syncthreads();  // waits for the loads first
    // from here base_a / base_b point at stage 3

    // lane's LDS byte addresses of its fragments for (ring slot 0, block 0), step 0 and step 1: row r's chunk c is
    // in 16-byte slot 4 r + (c ^ ((r >> 2) & 3)); lanes 0..31 take a step's first chunk, lanes 32..63 the second
    const unsigned a_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)&sm.a[0][0];
    const unsigned b_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)&sm.b[0][0];
    const unsigned turn = (unsigned)((l32 >> 2) & 3);
    unsigned a_addr[2], b_addr[2];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const unsigned chunk = (unsigned)(2 * st + half) ^ turn;
      a_addr[st] = a_lds + ((wm * 128 + l32) * 4 + chunk) * 16;
      b_addr[st] = b_lds + ((wn * 128 + l32) * 4 + chunk) * 16;
    }
    const unsigned m0_a0 = __builtin_amdgcn_readfirstlane(a_lds + wave * 4096);
    const unsigned m0_b0 = __builtin_amdgcn_readfirstlane(b_lds + wave * 4096);
    typedef Loop L;
    L::prime(r, a_addr, b_addr);
    int stage = 0;
    for (int t = 0; t < nstages; ++t) {
      const int next = (stage + 1) & 3, slot3 = (stage + 3) & 3;
      L::tile(r, a_addr, b_addr, (unsigned)((next - stage) * (int)PANEL), nstages - (t + 3),
              m0_a0 + slot3 * PANEL, m0_b0 + slot3 * PANEL, off_a, off_b, base_a, base_b);
      base_a += STAGE_K_BYTES;
      base_b += STAGE_K_BYTES;
      stage = next;
    }
    // the compiler does not see the matrix instructions inside the statements, so it cannot know that the
    // accumulators it reads next may still be on their way: the last one written needs 18 wait states
    asm volatile("s_nop 15\ns_nop 7" : CUASR_NARROW_ACC);
  }

  // ---- epilogue.  Block (bi, bj), register e of lane l: row 8 * (e / 4) + 4 * (l / 32) + e % 4, column l % 32: a
  // store instruction writes 128 consecutive bytes of two rows.  The four blocks of a block row are stored register
  // by register, so that four consecutive instructions write 512 consecutive bytes of each of their two rows: block
  // by block (sixteen instructions that touch 32 rows before the next 128 bytes of any of them follow) the same
  // stores took 10 us longer per round of tiles at 4096 x 4096, a third of an int8 launch with 64 bytes of k.  (With
  // the operands of the matrix instruction swapped a lane holds four consecutive columns per group of registers and
  // stores vectors -- a quarter of the store instructions, but each touching 32 rows, a leading dimension apart:
  // measured 25 % slower at 8192^3.)
  const EpilogueScalars<Result> sc = resolve_scalars<Result>(p, kMultiplies);
  const Result *C = reinterpret_cast<const Result *>(p.C);
  Result *D = reinterpret_cast<Result *>(p.D);
  const int col0 = n0 + wn * 128 + l32;
  // one copy of the stores per case (partial sums for a split-K workspace; results with and without a source), the
  // case chosen once: with the tests inside, per element, the same stores took 3 us longer per tile
  auto store_all = [&](auto to_workspace, auto with_source) {
    constexpr bool WS = decltype(to_workspace)::value, SRC = decltype(with_source)::value;
    auto row_of = [&](int bi, int e) { return (long long)(m0 + wm * 128 + bi * 32 + 8 * (e / 4) + 4 * half + (e % 4)); };
    // a block row's 64 source elements are requested together (D may be C, so the compiler cannot move a load of C
    // above a store to D by itself: one load at a time, each waited for, made this epilogue as long as the
    // product), and the next block row's before this one's results are stored, so that the trip to memory is
    // waited for once, not four times (a thread reads exactly the elements it writes, later)
    Result src[2][16][4];
    auto request = [&](int bi) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int bj = 0; bj < 4; ++bj) src[bi & 1][e][bj] = C[row_of(bi, e) * p.ldc + col0 + bj * 32];
    };
    if constexpr (SRC) request(0);
#pragma unroll
    for (int bi = 0; bi < 4; ++bi) {
      if constexpr (SRC) {
        if (bi + 1 < 4) request(bi + 1);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int bj = 0; bj < 4; ++bj) {
          const long long row = row_of(bi, e);
          const int col = col0 + bj * 32;
          const int blk = 4 * bi + bj;
          const int bits = r.acc[blk / 2][(blk % 2) * 16 + e];
          if constexpr (WS) {
            reinterpret_cast<int32_t *>(p.workspace)[((long long)blockIdx.y * p.m + row) * p.n + col] = bits;
          } else {
            // unsigned arithmetic: the same bits as the two's-complement result, with no overflow to reason about
            uint32_t out = (uint32_t)sc.alpha * (uint32_t)bits;
            if constexpr (SRC) out += (uint32_t)sc.beta * (uint32_t)src[bi & 1][e][bj];
            D[row * p.ldd + col] = (int32_t)out;
          }
        }
    }
  };
  if (p.workspace) store_all(std::true_type{}, std::false_type{});
  else if (sc.source_needed) store_all(std::false_type{}, std::true_type{});
  else store_all(std::false_type{}, std::false_type{});
}

// ---- binary16 on v_mfma_f32_16x16x32_f16.  On random binary16 operands the chip delivers 2.07 PFLOP/s through this
// shape and 1.68 through 32 x 32 x 16 (loops of the bare instructions on register contents, both at the board's power
// cap; for int8 it is the other way round, 3.26 against 2.99 POP/s), so binary16 takes this kernel.  Same tile, ring
// and loads; what differs: the instruction takes 64 bytes of k per row, so a stage is one step of 64 matrix
// instructions on 8 x 8 blocks of 16 x 16; lane l supplies row (column) l % 16, bytes 16 (l / 16) .. + 15 of the
// stage's 64, so a fragment read covers 16 rows x 4 chunks, which reads without bank conflicts when row r's chunk
// c lies in slot 4 r + (c ^ ((r >> 1) & 3)); fragments are double-buffered by stage (two forms of the generated
// statement, alternated); register e of block (bi, bj) holds row 4 (l / 16) + e, column l % 16.
struct Regs16 {
  asm_v32 acc[8];    // a0 .. a255: block (bm, bn) in a[4 (8 bm + bn) : +3]
  asm_v32 frag[4];   // v0 .. v127: buffer u, A block b in v[64 u + 4 b : +3], B block b in v[64 u + 32 + 4 b : +3]
};
#define CUASR_NARROW16_FRAG "+{v[0:31]}"(r.frag[0]), "+{v[32:63]}"(r.frag[1]), "+{v[64:95]}"(r.frag[2]), "+{v[96:127]}"(r.frag[3])
// what a stage's part of a statement takes: where the fragment addresses move to, how many stages are left to fetch,
// the ring slot and the global address of the stage three ahead
struct Stage16 {
  unsigned step;
  int fetch;
  unsigned m0_a, m0_b;
  const char *base_a, *base_b;
};
#define CUASR_NARROW16_STAGE(n, s)                                                                                        \
  [step##n] "s"(s.step), [fetch##n] "s"(s.fetch), [m0_a##n] "s"(s.m0_a), [m0_b##n] "s"(s.m0_b), [base_a##n] "s"(s.base_a), \
      [base_b##n] "s"(s.base_b)
#define CUASR_NARROW16_OUT                                                                                                \
  CUASR_NARROW_ACC, CUASR_NARROW16_FRAG, [a_addr] "+v"(a_addr), [b_addr] "+v"(b_addr), [m0_save] "=&s"(m0_save)
#define CUASR_NARROW16_OFFS                                                                                               \
  [off_a0] "v"(off_a[0]), [off_a1] "v"(off_a[1]), [off_a2] "v"(off_a[2]), [off_a3] "v"(off_a[3]),                         \
      [off_b0] "v"(off_b[0]), [off_b1] "v"(off_b[1]), [off_b2] "v"(off_b[2]), [off_b3] "v"(off_b[3])
struct Loop16 {
  static __device__ __forceinline__ void prime(Regs16 &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_n16_f16_prime.inc"
        : CUASR_NARROW16_FRAG : [a_addr] "v"(a_addr), [b_addr] "v"(b_addr) : "memory");
  }
  // two stages (the first in fragment buffer 0, the second in buffer 1)
  static __device__ __forceinline__ void pair(Regs16 &r, unsigned &a_addr, unsigned &b_addr, const Stage16 &s0, const Stage16 &s1,
                                              const unsigned (&off_a)[4], const unsigned (&off_b)[4]) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_n16_f16_pair.inc"
        : CUASR_NARROW16_OUT
        : CUASR_NARROW16_STAGE(0, s0), CUASR_NARROW16_STAGE(1, s1), CUASR_NARROW16_OFFS
        : "scc", "memory");
  }
  // one stage (in buffer 0): an odd last one
  static __device__ __forceinline__ void single(Regs16 &r, unsigned &a_addr, unsigned &b_addr, const Stage16 &s0,
                                                const unsigned (&off_a)[4], const unsigned (&off_b)[4]) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_n16_f16_tile0.inc"
        : CUASR_NARROW16_OUT
        : CUASR_NARROW16_STAGE(0, s0), CUASR_NARROW16_OFFS
        : "scc", "memory");
  }
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mfma_narrow_kernel16(Problem p) {
  constexpr long long E = sizeof(half_t);
  __shared__ __attribute__((aligned(1024))) Smem sm;
  select_batch<half_t, half_t>(p);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l16 = lane & 15, quarter = lane >> 4;
  const int tiles_m = p.m / BM, tiles_n = p.n / BN;   // the host sends whole tiles only
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const int nstages = (int)((long long)p.k * E / STAGE_K_BYTES);   // (the host sends whole stages only)

  Regs16 r;
#pragma unroll
  for (int v = 0; v < 8; ++v) r.acc[v] = asm_v32(0);
#pragma unroll
  for (int v = 0; v < 4; ++v) r.frag[v] = asm_v32(0);

  if (nstages > 0) {
    const char *base_a = reinterpret_cast<const char *>(p.A) + (long long)m0 * p.sa_m * E;
    const char *base_b = reinterpret_cast<const char *>(p.B) + (long long)n0 * p.sb_n * E;
    // this wave's 64 rows of each panel in four loads of 16 rows x 64 bytes: lane l of load h fetches row
    // 64 wave + 16 h + l / 4, chunk (l % 4) ^ ((l / 8) % 4) -- the chunk that belongs in the LDS slot the lane writes
    unsigned off_a[4], off_b[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const long long row = wave * 64 + 16 * h + lane / 4;
      const unsigned chunk = (unsigned)((lane & 3) ^ ((lane >> 3) & 3));
      off_a[h] = (unsigned)(row * p.sa_m * E) + 16u * chunk;
      off_b[h] = (unsigned)(row * p.sb_n * E) + 16u * chunk;
    }
    auto fetch = [&](int stage) {
#pragma unroll
      for (int h = 0; h < 4; ++h) dma16(base_a + off_a[h], &sm.a[stage][(wave * 4 + h) * 1024]);
#pragma unroll
      for (int h = 0; h < 4; ++h) dma16(base_b + off_b[h], &sm.b[stage][(wave * 4 + h) * 1024]);
    };
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      if (s < nstages) fetch(s);
      base_a += STAGE_K_BYTES;
      base_b += STAGE_K_BYTES;
    }
    __syncthreads();  // waits for the loads first
    // from here base_a / base_b point at stage 3

    const unsigned a_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)&sm.a[0][0];
    const unsigned b_lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)&sm.b[0][0];
    const unsigned chunk = (unsigned)quarter ^ (unsigned)((l16 >> 1) & 3);
    unsigned a_addr = a_lds + ((wm * 128 + l16) * 4 + chunk) * 16;
    unsigned b_addr = b_lds + ((wn * 128 + l16) * 4 + chunk) * 16;
    const unsigned m0_a0 = __builtin_amdgcn_readfirstlane(a_lds + wave * 4096);
    const unsigned m0_b0 = __builtin_amdgcn_readfirstlane(b_lds + wave * 4096);
    Loop16::prime(r, a_addr, b_addr);
    // two stages per statement: the statements pin 384 registers, which pass from one turn of the loop to the next
    // without copies only when the loop holds a single statement
    int stage = 0, t = 0;
    auto next_stage = [&]() {
      const int next = (stage + 1) & 3, slot3 = (stage + 3) & 3;
      const Stage16 s{(unsigned)((next - stage) * (int)PANEL), nstages - (t + 3), m0_a0 + slot3 * PANEL, m0_b0 + slot3 * PANEL, base_a, base_b};
      base_a += STAGE_K_BYTES;
      base_b += STAGE_K_BYTES;
      stage = next;
      ++t;
      return s;
    };
    while (t + 1 < nstages) {
      const Stage16 s0 = next_stage(), s1 = next_stage();
      Loop16::pair(r, a_addr, b_addr, s0, s1, off_a, off_b);
    }
    if (t < nstages) {
      const Stage16 s0 = next_stage();
      Loop16::single(r, a_addr, b_addr, s0, off_a, off_b);
    }
    // the compiler does not see the matrix instructions inside the statements, so it cannot know that the
    // accumulators it reads next may still be on their way
    asm volatile("s_nop 15\ns_nop 7" : CUASR_NARROW_ACC);
  }

  // ---- epilogue.  A store instruction writes 32 consecutive bytes of four rows; a block row's eight blocks are
  // stored register by register (eight consecutive instructions write 256 consecutive bytes of each of their four
  // rows), its sources requested together and one block row ahead (see the kernel above).
  const EpilogueScalars<half_t> sc = resolve_scalars<half_t>(p, kMultiplies);
  const half_t *C = reinterpret_cast<const half_t *>(p.C);
  half_t *D = reinterpret_cast<half_t *>(p.D);
  const int col0 = n0 + wn * 128 + l16;
  auto store_all = [&](auto with_source) {
    constexpr bool SRC = decltype(with_source)::value;
    auto row_of = [&](int bi, int e) { return (long long)(m0 + wm * 128 + bi * 16 + 4 * quarter + e); };
    half_t src[2][4][8];
    auto request = [&](int bi) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int bj = 0; bj < 8; ++bj) src[bi & 1][e][bj] = C[row_of(bi, e) * p.ldc + col0 + bj * 16];
    };
    if constexpr (SRC) request(0);
#pragma unroll
    for (int bi = 0; bi < 8; ++bi) {
      if constexpr (SRC) {
        if (bi + 1 < 8) request(bi + 1);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int bj = 0; bj < 8; ++bj) {
          const int idx = 4 * (8 * bi + bj) + e;
          // D = alpha * acc + beta * C in float, rounded to binary16 once
          float out = float(sc.alpha) * __builtin_bit_cast(float, (int)r.acc[idx / 32][idx % 32]);
          if constexpr (SRC) out += float(sc.beta) * float(src[bi & 1][e][bj]);
          D[row_of(bi, e) * p.ldd + col0 + bj * 16] = half_t(out);
        }
    }
  };
  if (sc.source_needed) store_all(std::true_type{});
  else store_all(std::false_type{});
}

// ---- the same with the panels fetched 128 bytes of k per row, for k ranges that are whole stages of 128 bytes.  Eight
// neighbouring lanes of a load fetch the eight 16-byte chunks of one row's 128 bytes -- a whole cache line per
// request to L2, where the 64-byte stages above make two requests of it, and requests, not bytes, are what that path
// runs out of (a build whose loads merely had this shape, with wrong results, ran 6 % faster at 4096^3 and 8192^3).
// A stage is then two steps of the matrix instruction; the ring holds five units of one operand's 256 rows x 128
// bytes (all 160 KiB of LDS): the A and B panels of this stage and of the next, and the A panel after that.  A's
// panel of stage s is unit 2 s, B's unit 2 s + 1, unit u lives in slot u % 5; once every wave holds stage t's
// fragments its two slots take the B panel two stages ahead and the A panel three ahead.  Row r's chunk c lies in
// 16-byte position 8 r + (c ^ (r & 7)), which keeps both the loads' writes (consecutive positions) and the fragment
// reads (16 rows x 4 chunks) free of bank conflicts.
constexpr int LINE_K_BYTES = 128, UNITS = 5;
constexpr unsigned UNIT = LINE_K_BYTES * 256;   // 32 KiB
struct SmemLine {
  unsigned char unit[UNITS][UNIT];
};
struct StageLine {
  unsigned a_step, b_step;   // where the fragment addresses move to
  int fetch_x, fetch_y;      // > 0: the B panel two stages ahead / the A panel three ahead exists
  unsigned m0_x, m0_y;       // this wave's part of the slots they go to
  const char *base_x, *base_y;
};
struct LoopLine16 {
  static __device__ __forceinline__ void prime(Regs16 &r, unsigned a_addr0, unsigned b_addr0) {
    asm volatile(
#include "gen/mfma_asm_n16l_f16_prime.inc"
        : CUASR_NARROW16_FRAG : [a_addr0] "v"(a_addr0), [b_addr0] "v"(b_addr0) : "memory");
  }
  static __device__ __forceinline__ void tile(Regs16 &r, unsigned (&a_addr)[2], unsigned (&b_addr)[2], const StageLine &s,
                                              const unsigned (&off_a)[8], const unsigned (&off_b)[8]) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_n16l_f16_tile.inc"
        : CUASR_NARROW_ACC, CUASR_NARROW16_FRAG, [a_addr0] "+v"(a_addr[0]), [a_addr1] "+v"(a_addr[1]), [b_addr0] "+v"(b_addr[0]),
          [b_addr1] "+v"(b_addr[1]), [m0_save] "=&s"(m0_save)
        : [a_step] "s"(s.a_step), [b_step] "s"(s.b_step), [fetch_x] "s"(s.fetch_x), [fetch_y] "s"(s.fetch_y), [m0_x] "s"(s.m0_x),
          [m0_y] "s"(s.m0_y), [base_x] "s"(s.base_x), [base_y] "s"(s.base_y),
          [off_a0] "v"(off_a[0]), [off_a1] "v"(off_a[1]), [off_a2] "v"(off_a[2]), [off_a3] "v"(off_a[3]), [off_a4] "v"(off_a[4]),
          [off_a5] "v"(off_a[5]), [off_a6] "v"(off_a[6]), [off_a7] "v"(off_a[7]),
          [off_b0] "v"(off_b[0]), [off_b1] "v"(off_b[1]), [off_b2] "v"(off_b[2]), [off_b3] "v"(off_b[3]), [off_b4] "v"(off_b[4]),
          [off_b5] "v"(off_b[5]), [off_b6] "v"(off_b[6]), [off_b7] "v"(off_b[7])
        : "scc", "memory");
  }
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mfma_narrow_kernel16_lines(Problem p) {
  constexpr long long E = sizeof(half_t);
  __shared__ __attribute__((aligned(1024))) SmemLine sm;
  select_batch<half_t, half_t>(p);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l16 = lane & 15, quarter = lane >> 4;
  const int tiles_m = p.m / BM, tiles_n = p.n / BN;   // the host sends whole tiles only
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const int nstages = (int)((long long)p.k * E / LINE_K_BYTES);   // (the host sends whole stages only)

  Regs16 r;
#pragma unroll
  for (int v = 0; v < 8; ++v) r.acc[v] = asm_v32(0);
#pragma unroll
  for (int v = 0; v < 4; ++v) r.frag[v] = asm_v32(0);

  if (nstages > 0) {
    const char *panel_a = reinterpret_cast<const char *>(p.A) + (long long)m0 * p.sa_m * E;
    const char *panel_b = reinterpret_cast<const char *>(p.B) + (long long)n0 * p.sb_n * E;
    // this wave's 64 rows of a unit in eight loads of 8 rows x 128 bytes: lane l of load h fetches row
    // 64 wave + 8 h + l / 8, chunk (l % 8) ^ (l / 8) -- the chunk that belongs in the position the lane writes
    unsigned off_a[8], off_b[8];
#pragma unroll
    for (int h = 0; h < 8; ++h) {
      const long long row = wave * 64 + 8 * h + lane / 8;
      const unsigned chunk = (unsigned)((lane & 7) ^ ((lane >> 3) & 7));
      off_a[h] = (unsigned)(row * p.sa_m * E) + 16u * chunk;
      off_b[h] = (unsigned)(row * p.sb_n * E) + 16u * chunk;
    }
    auto fetch = [&](const char *base, const unsigned (&off)[8], int slot) {
#pragma unroll
      for (int h = 0; h < 8; ++h) dma16(base + off[h], &sm.unit[slot][(wave * 8 + h) * 1024]);
    };
    // units 0 .. 4: A0 B0 A1 B1 A2
    fetch(panel_a, off_a, 0);
    fetch(panel_b, off_b, 1);
    if (nstages > 1) {
      fetch(panel_a + LINE_K_BYTES, off_a, 2);
      fetch(panel_b + LINE_K_BYTES, off_b, 3);
    }
    if (nstages > 2) fetch(panel_a + 2 * LINE_K_BYTES, off_a, 4);
    __syncthreads();  // waits for the loads first

    const unsigned lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)&sm.unit[0][0];
    unsigned a_addr[2], b_addr[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const unsigned chunk = (unsigned)(4 * h + quarter) ^ (unsigned)(l16 & 7);
      a_addr[h] = lds + ((wm * 128 + l16) * 8 + chunk) * 16;          // A's first panel: slot 0
      b_addr[h] = lds + UNIT + ((wn * 128 + l16) * 8 + chunk) * 16;   // B's: slot 1
    }
    const unsigned m0_wave = __builtin_amdgcn_readfirstlane(lds + wave * 8192);
    LoopLine16::prime(r, a_addr[0], b_addr[0]);
    int ua = 0, ub = 1;   // the slots of this stage's panels
    for (int t = 0; t < nstages; ++t) {
      const int na = (ua + 2) % UNITS, nb = (ub + 2) % UNITS;
      const StageLine s{(unsigned)((na - ua) * (int)UNIT), (unsigned)((nb - ub) * (int)UNIT), nstages - (t + 2), nstages - (t + 3),
                        m0_wave + ua * UNIT, m0_wave + ub * UNIT, panel_b + (long long)(t + 2) * LINE_K_BYTES,
                        panel_a + (long long)(t + 3) * LINE_K_BYTES};
      LoopLine16::tile(r, a_addr, b_addr, s, off_a, off_b);
      ua = na;
      ub = nb;
    }
    // the compiler does not see the matrix instructions inside the statements, so it cannot know that the
    // accumulators it reads next may still be on their way
    asm volatile("s_nop 15\ns_nop 7" : CUASR_NARROW_ACC);
  }

  // ---- epilogue (that of mfma_narrow_kernel16)
  const EpilogueScalars<half_t> sc = resolve_scalars<half_t>(p, kMultiplies);
  const half_t *C = reinterpret_cast<const half_t *>(p.C);
  half_t *D = reinterpret_cast<half_t *>(p.D);
  const int col0 = n0 + wn * 128 + l16;
  auto store_all = [&](auto with_source) {
    constexpr bool SRC = decltype(with_source)::value;
    auto row_of = [&](int bi, int e) { return (long long)(m0 + wm * 128 + bi * 16 + 4 * quarter + e); };
    half_t src[2][4][8];
    auto request = [&](int bi) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int bj = 0; bj < 8; ++bj) src[bi & 1][e][bj] = C[row_of(bi, e) * p.ldc + col0 + bj * 16];
    };
    if constexpr (SRC) request(0);
#pragma unroll
    for (int bi = 0; bi < 8; ++bi) {
      if constexpr (SRC) {
        if (bi + 1 < 8) request(bi + 1);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int bj = 0; bj < 8; ++bj) {
          const int idx = 4 * (8 * bi + bj) + e;
          float out = float(sc.alpha) * __builtin_bit_cast(float, (int)r.acc[idx / 32][idx % 32]);
          if constexpr (SRC) out += float(sc.beta) * float(src[bi & 1][e][bj]);
          D[row_of(bi, e) * p.ldd + col0 + bj * 16] = half_t(out);
        }
    }
  };
  if (sc.source_needed) store_all(std::true_type{});
  else store_all(std::false_type{});
}

// ---- int8 with the panels fetched 128 bytes of k per row (the ring of five one-operand units of
// mfma_narrow_kernel16_lines; a stage is four steps of the 32 x 32 x 32 instruction).  A fragment read covers 32 rows x
// 2 chunks here, which reads without bank conflicts when row r's chunk c lies in position 8 r + (c ^ ((r >> 1) & 7)).
struct LoopLineI8 {
  static __device__ __forceinline__ void prime(Regs &r, unsigned a_addr0, unsigned b_addr0) {
    asm volatile(
#include "gen/mfma_asm_nl_i8_prime.inc"
        : "+{v[0:31]}"(r.frag[0]), "+{v[32:63]}"(r.frag[1]) : [a_addr0] "v"(a_addr0), [b_addr0] "v"(b_addr0) : "memory");
  }
  static __device__ __forceinline__ void tile(Regs &r, unsigned (&a_addr)[4], unsigned (&b_addr)[4], const StageLine &s,
                                              const unsigned (&off_a)[8], const unsigned (&off_b)[8]) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_nl_i8_tile.inc"
        : CUASR_NARROW_ACC, "+{v[0:31]}"(r.frag[0]), "+{v[32:63]}"(r.frag[1]), [a_addr0] "+v"(a_addr[0]), [a_addr1] "+v"(a_addr[1]),
          [a_addr2] "+v"(a_addr[2]), [a_addr3] "+v"(a_addr[3]), [b_addr0] "+v"(b_addr[0]), [b_addr1] "+v"(b_addr[1]),
          [b_addr2] "+v"(b_addr[2]), [b_addr3] "+v"(b_addr[3]), [m0_save] "=&s"(m0_save)
        : [a_step] "s"(s.a_step), [b_step] "s"(s.b_step), [fetch_x] "s"(s.fetch_x), [fetch_y] "s"(s.fetch_y), [m0_x] "s"(s.m0_x),
          [m0_y] "s"(s.m0_y), [base_x] "s"(s.base_x), [base_y] "s"(s.base_y),
          [off_a0] "v"(off_a[0]), [off_a1] "v"(off_a[1]), [off_a2] "v"(off_a[2]), [off_a3] "v"(off_a[3]), [off_a4] "v"(off_a[4]),
          [off_a5] "v"(off_a[5]), [off_a6] "v"(off_a[6]), [off_a7] "v"(off_a[7]),
          [off_b0] "v"(off_b[0]), [off_b1] "v"(off_b[1]), [off_b2] "v"(off_b[2]), [off_b3] "v"(off_b[3]), [off_b4] "v"(off_b[4]),
          [off_b5] "v"(off_b[5]), [off_b6] "v"(off_b[6]), [off_b7] "v"(off_b[7])
        : "scc", "memory");
  }
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mfma_narrow_kernel_lines(Problem p) {
  __shared__ __attribute__((aligned(1024))) SmemLine sm;
  select_batch<int32_t, int8_t>(p);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, half = lane >> 5, l32 = lane & 31;
  const int tiles_m = p.m / BM, tiles_n = p.n / BN;   // the host sends whole tiles only
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const int nstages = p.k / LINE_K_BYTES;   // (the host sends whole stages only, and no split-K slices)

  Regs r;
#pragma unroll
  for (int v = 0; v < 8; ++v) r.acc[v] = asm_v32(0);
#pragma unroll
  for (int v = 0; v < 2; ++v) r.frag[v] = asm_v32(0);

  if (nstages > 0) {
    const char *panel_a = reinterpret_cast<const char *>(p.A) + (long long)m0 * p.sa_m;
    const char *panel_b = reinterpret_cast<const char *>(p.B) + (long long)n0 * p.sb_n;
    // this wave's 64 rows of a unit in eight loads of 8 rows x 128 bytes: lane l of load h fetches row
    // R = 64 wave + 8 h + l / 8, chunk (l % 8) ^ ((R >> 1) & 7) -- the chunk that belongs in the position the lane writes
    unsigned off_a[8], off_b[8];
#pragma unroll
    for (int h = 0; h < 8; ++h) {
      const long long row = wave * 64 + 8 * h + lane / 8;
      const unsigned chunk = (unsigned)((lane & 7) ^ (int)((row >> 1) & 7));
      off_a[h] = (unsigned)(row * p.sa_m) + 16u * chunk;
      off_b[h] = (unsigned)(row * p.sb_n) + 16u * chunk;
    }
    auto fetch = [&](const char *base, const unsigned (&off)[8], int slot) {
#pragma unroll
      for (int h = 0; h < 8; ++h) dma16(base + off[h], &sm.unit[slot][(wave * 8 + h) * 1024]);
    };
    // units 0 .. 4: A0 B0 A1 B1 A2
    fetch(panel_a, off_a, 0);
    fetch(panel_b, off_b, 1);
    if (nstages > 1) {
      fetch(panel_a + LINE_K_BYTES, off_a, 2);
      fetch(panel_b + LINE_K_BYTES, off_b, 3);
    }
    if (nstages > 2) fetch(panel_a + 2 * LINE_K_BYTES, off_a, 4);
    __syncthreads();  // waits for the loads first

    const unsigned lds = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)&sm.unit[0][0];
    unsigned a_addr[4], b_addr[4];
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      const unsigned chunk = (unsigned)(2 * st + half) ^ (unsigned)((l32 >> 1) & 7);
      a_addr[st] = lds + ((wm * 128 + l32) * 8 + chunk) * 16;          // A's first panel: slot 0
      b_addr[st] = lds + UNIT + ((wn * 128 + l32) * 8 + chunk) * 16;   // B's: slot 1
    }
    const unsigned m0_wave = __builtin_amdgcn_readfirstlane(lds + wave * 8192);
    LoopLineI8::prime(r, a_addr[0], b_addr[0]);
    int ua = 0, ub = 1;   // the slots of this stage's panels
    for (int t = 0; t < nstages; ++t) {
      const int na = (ua + 2) % UNITS, nb = (ub + 2) % UNITS;
      const StageLine s{(unsigned)((na - ua) * (int)UNIT), (unsigned)((nb - ub) * (int)UNIT), nstages - (t + 2), nstages - (t + 3),
                        m0_wave + ua * UNIT, m0_wave + ub * UNIT, panel_b + (long long)(t + 2) * LINE_K_BYTES,
                        panel_a + (long long)(t + 3) * LINE_K_BYTES};
      LoopLineI8::tile(r, a_addr, b_addr, s, off_a, off_b);
      ua = na;
      ub = nb;
    }
    // the compiler does not see the matrix instructions inside the statements, so it cannot know that the
    // accumulators it reads next may still be on their way: the last one written needs 18 wait states
    asm volatile("s_nop 15\ns_nop 7" : CUASR_NARROW_ACC);
  }

  // ---- epilogue (that of mfma_narrow_kernel, without the split-K case)
  const EpilogueScalars<int32_t> sc = resolve_scalars<int32_t>(p, kMultiplies);
  const int32_t *C = reinterpret_cast<const int32_t *>(p.C);
  int32_t *D = reinterpret_cast<int32_t *>(p.D);
  const int col0 = n0 + wn * 128 + l32;
  auto store_all = [&](auto with_source) {
    constexpr bool SRC = decltype(with_source)::value;
    auto row_of = [&](int bi, int e) { return (long long)(m0 + wm * 128 + bi * 32 + 8 * (e / 4) + 4 * half + (e % 4)); };
    int32_t src[2][16][4];
    auto request = [&](int bi) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int bj = 0; bj < 4; ++bj) src[bi & 1][e][bj] = C[row_of(bi, e) * p.ldc + col0 + bj * 32];
    };
    if constexpr (SRC) request(0);
#pragma unroll
    for (int bi = 0; bi < 4; ++bi) {
      if constexpr (SRC) {
        if (bi + 1 < 4) request(bi + 1);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int bj = 0; bj < 4; ++bj) {
          const int blk = 4 * bi + bj;
          const int bits = r.acc[blk / 2][(blk % 2) * 16 + e];
          // unsigned arithmetic: the same bits as the two's-complement result, with no overflow to reason about
          uint32_t out = (uint32_t)sc.alpha * (uint32_t)bits;
          if constexpr (SRC) out += (uint32_t)sc.beta * (uint32_t)src[bi & 1][e][bj];
          D[row_of(bi, e) * p.ldd + col0 + bj * 32] = (int32_t)out;
        }
    }
  };
  if (sc.source_needed) store_all(std::true_type{});
  else store_all(std::false_type{});
}

// whole tiles, whole stages, both operands k-contiguous with 16-byte aligned rows, a panel's 256 rows within 32
// bits of byte offset
static bool can_run(const Problem &p, long long esize) {
  auto al16 = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  if (p.sa_k != 1 || p.sb_k != 1 || p.m <= 0 || p.n <= 0 || p.k <= 0) return false;
  if (p.m % BM || p.n % BN || (p.k * esize) % STAGE_K_BYTES) return false;
  if (p.workspace && (p.k_per_slice * esize) % STAGE_K_BYTES) return false;
  if ((p.sa_m * esize) % 16 || (p.sb_n * esize) % 16 || !al16(p.A) || !al16(p.B)) return false;
  if (256 * p.sa_m * esize >= (1LL << 32) || 256 * p.sb_n * esize >= (1LL << 32)) return false;
  if (p.batch > 1 && ((p.batch_a * esize) % 16 || (p.batch_b * esize) % 16)) return false;
  return true;
}

template <bool I8> static hipError_t launch(const Problem &p, hipStream_t s) {
  const long long tiles = (long long)(p.m / BM) * (p.n / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  const dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1, p.batch), block(256);
  if constexpr (I8) {
    // whole stages of 128 bytes (and no split-K slices) take the form that fetches whole cache lines: 4096^3 82.5 -> 79.5 us,
    // 6144^3 283 -> 274 us, 8192^3 620 -> 573 us
    if (!p.workspace && p.k % LINE_K_BYTES == 0) launch_kernel(mfma_narrow_kernel_lines, grid, block, 0, s, p);
    else launch_kernel(mfma_narrow_kernel, grid, block, 0, s, p);
  } else {
    // whole stages of 128 bytes take the form that fetches whole cache lines, up to three rounds of workgroups: 4096^3
    // 118.8 -> 112.2 us, 6144^3 448 -> 434 us; from 8192^3 on (four rounds, at the board's power cap either way) it is
    // 1 - 2 % behind
    static const int units = [] {
      int dev = 0, n = 0;
      if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) (void)hipGetLastError();
      return n > 0 ? n : 256;
    }();
    const long long groups = tiles * (long long)p.batch;
    if ((p.k * 2) % LINE_K_BYTES == 0 && groups <= 3LL * units) launch_kernel(mfma_narrow_kernel16_lines, grid, block, 0, s, p);
    else launch_kernel(mfma_narrow_kernel16, grid, block, 0, s, p);
  }
  return take_launch_status();
}

}  // namespace mfma_narrow

// One wave per SIMD and one workgroup per compute unit: a launch takes ceil(workgroups / compute units) tile
// times, so the hand-scheduled tile is for launches that fill most of their last such round; smaller or oddly
// sized ones are better served by the compiled kernels' 128 x 128 tiles, two per compute unit.
static bool narrow_fills(const Problem &p, int units) {
  if (units <= 0) units = 256;
  const long long groups = (long long)(p.m / mfma_narrow::BM) * (p.n / mfma_narrow::BN) * (p.workspace ? p.slices : 1) * p.batch;
  const long long rounds = (groups + units - 1) / units;
  return groups * 4 >= rounds * units * 3;
}

bool mfma_narrow_i8_can_run(const Problem &p, int units) { return mfma_narrow::can_run(p, 1) && narrow_fills(p, units); }
bool mfma_narrow_f16_can_run(const Problem &p, int units) { return !p.workspace && mfma_narrow::can_run(p, 2) && narrow_fills(p, units); }
hipError_t launch_mfma_narrow_i8(const Problem &p, hipStream_t s) { return mfma_narrow::launch<true>(p, s); }
hipError_t launch_mfma_narrow_f16(const Problem &p, hipStream_t s) { return mfma_narrow::launch<false>(p, s); }

}  // namespace cuasr_amd
