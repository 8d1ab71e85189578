// plus-times for double on the matrix cores, hand-scheduled:
//     D = alpha * (A . B) + beta * C      with v_mfma_f64_16x16x4_f64
//
// The fast form of mfma_gemm_f64.hip (same instruction, same output tile 128 x 128, same accumulator layout,
// same place in the library: the reference's SIMT kernel include/cuasr/gemm/kernel/srgemm.h:156-321 for
// DefaultSemiRingConfiguration<plus<double>, multiplies<double>>) for products whose k range is a multiple of 16
// and whose operands the direct-to-LDS loads can fetch (16-byte aligned rows).  As in mfma_direct_f32.hip:
// panels go global -> LDS without passing registers, the main loop is one generated asm statement per k-tile
// (gen_direct_asm.py, Mfma64Body: 64 matrix instructions with the LDS reads and the loads spread between
// them, one wait, one barrier), and a period of 8 k is walked so that a k-contiguous panel ([k/2][X][2] in LDS,
// the image the loads produce) feeds a 16-row block's two steps with one 16-byte read.  Two LDS stages of 32 KiB
// (two workgroups per compute unit): the loads of the tile two ahead are issued right after the barrier in the
// middle of a tile, where the stage they go to has been read for the last time.
// The sum over k is formed in the instruction's order, so results agree with the host reference to rounding
// (|d - r| <= 1e-12 * sum_k |a||b|), like the compiled form.
#include "semiring.h"

namespace cuasr_amd {
namespace gemm_mfma_direct_f64 {

constexpr int BM = 128, BN = 128, BK = 16, STAGES = 2;
constexpr unsigned A_STAGE = BK * BM * 8, B_STAGE = BK * BN * 8;

struct Smem {
  double a[STAGES][BK * BM];
  double b[STAGES][BK * BN];
};

typedef float asm_v16 __attribute__((ext_vector_type(16)));
typedef double asm_d8 __attribute__((ext_vector_type(8)));
struct Regs {
  asm_d8 acc[8];    // v0 .. v127: block (bm, bn) = four doubles at element 4 ((4 bm + bn) & 1) of acc[(4 bm + bn) / 2]
  asm_v16 frag[4];  // v128 .. v191
};

__device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int &bm, int &bn) {
  const int total = tiles_m * tiles_n;
  // consecutive workgroup ids land on consecutive XCDs (8, one L2 each): give every XCD one contiguous run
  if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
  constexpr int GROUP = 8;
  const int width = GROUP * tiles_n;
  const int group = id / width, first = group * GROUP;
  const int gsz = min(tiles_m - first, GROUP);
  bm = first + (id % width) % gsz;
  bn = (id % width) / gsz;
}

// The panel's LDS image has X * 8 positions of 16 bytes; a wave's load fills 64 consecutive ones.
//   k-contiguous: position = pair * X + x        (2 consecutive k of one x)
//   x-contiguous: position = k * (X / 2) + x2    (2 consecutive x at one k)
// x is clamped to the matrix edge: what clamped positions fetch is never stored.
template <bool KC, int X> __device__ __forceinline__ unsigned lane_offset(int pos, long long s_x, unsigned s_k_bytes, int x0, int x_end) {
  if constexpr (KC) return (unsigned)(min(x0 + (pos % X), x_end - 1) - x0) * (unsigned)s_x * 8u + (unsigned)(pos / X) * 16u;
  else return (unsigned)(min(x0 + (pos % (X / 2)) * 2, x_end - 2) - x0) * 8u + (unsigned)(pos / (X / 2)) * s_k_bytes;
}

__device__ __forceinline__ void dma16(const char *src, double *lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                   (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
}

#define CUASR_MFMA64_PRIME_OPERANDS                                                                                           \
        : "+{v[128:143]}"(r.frag[0]), "+{v[144:159]}"(r.frag[1]), "+{v[160:175]}"(r.frag[2]), "+{v[176:191]}"(r.frag[3])      \
        : [a_addr] "v"(a_addr), [b_addr] "v"(b_addr)                                                                          \
        : "memory"
#define CUASR_MFMA64_TILE_OPERANDS                                                                                            \
        : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]),                  \
          "+{v[64:79]}"(r.acc[4]), "+{v[80:95]}"(r.acc[5]), "+{v[96:111]}"(r.acc[6]), "+{v[112:127]}"(r.acc[7]),              \
          "+{v[128:143]}"(r.frag[0]), "+{v[144:159]}"(r.frag[1]), "+{v[160:175]}"(r.frag[2]), "+{v[176:191]}"(r.frag[3]),     \
          [a_addr] "+v"(a_addr), [b_addr] "+v"(b_addr), [m0_save] "=&s"(m0_save)                                              \
        : [a_step] "s"(a_step), [b_step] "s"(b_step), [fetch] "s"(fetch), [m0_a] "s"(m0_a), [m0_b] "s"(m0_b),                 \
          [off_a0] "v"(off[0]), [off_a1] "v"(off[1]), [off_a2] "v"(off[2]), [off_a3] "v"(off[3]), [off_b0] "v"(off[4]),       \
          [off_b1] "v"(off[5]), [off_b2] "v"(off[6]), [off_b3] "v"(off[7]), [base_a] "s"(base_a), [base_b] "s"(base_b)        \
        : "scc", "memory"
// prime: the fragments of the first 8 k into their registers; the tile must have landed in LDS stage 0.
// tile: one k-tile of 16 -- 64 matrix instructions per wave, the workgroup barrier that hands the LDS stage back, the
// fetch of the tile two ahead into it (if fetch > 0) and the fragments of the next tile's first 8 k.
#define CUASR_MFMA64_LOOP(AKC, BKC)                                                                                           \
  template <> struct Loop<AKC, BKC> {                                                                                         \
    static __device__ __forceinline__ void prime(Regs &r, unsigned a_addr, unsigned b_addr);                                  \
    static __device__ __forceinline__ void tile(Regs &r, unsigned &a_addr, unsigned &b_addr, unsigned a_step,                 \
                                                unsigned b_step, int fetch, unsigned m0_a, unsigned m0_b,                     \
                                                const unsigned (&off)[8], const char *base_a, const char *base_b);            \
  };

template <bool A_KC, bool B_KC> struct Loop;
CUASR_MFMA64_LOOP(true, false)
CUASR_MFMA64_LOOP(false, false)
CUASR_MFMA64_LOOP(false, true)
CUASR_MFMA64_LOOP(true, true)

#define CUASR_MFMA64_TILE_ARGS                                                                                                \
  Regs &r, unsigned &a_addr, unsigned &b_addr, unsigned a_step, unsigned b_step, int fetch, unsigned m0_a, unsigned m0_b,     \
      const unsigned (&off)[8], const char *base_a, const char *base_b

__device__ __forceinline__ void Loop<true, false>::prime(Regs &r, unsigned a_addr, unsigned b_addr) {
  asm volatile(
#include "gen/mfma_asm_md_kx_prime.inc"
      CUASR_MFMA64_PRIME_OPERANDS);
}
__device__ __forceinline__ void Loop<true, false>::tile(CUASR_MFMA64_TILE_ARGS) {
  unsigned m0_save;
  asm volatile(
#include "gen/mfma_asm_md_kx_tile.inc"
      CUASR_MFMA64_TILE_OPERANDS);
}
__device__ __forceinline__ void Loop<false, false>::prime(Regs &r, unsigned a_addr, unsigned b_addr) {
  asm volatile(
#include "gen/mfma_asm_md_xx_prime.inc"
      CUASR_MFMA64_PRIME_OPERANDS);
}
__device__ __forceinline__ void Loop<false, false>::tile(CUASR_MFMA64_TILE_ARGS) {
  unsigned m0_save;
  asm volatile(
#include "gen/mfma_asm_md_xx_tile.inc"
      CUASR_MFMA64_TILE_OPERANDS);
}
__device__ __forceinline__ void Loop<false, true>::prime(Regs &r, unsigned a_addr, unsigned b_addr) {
  asm volatile(
#include "gen/mfma_asm_md_xk_prime.inc"
      CUASR_MFMA64_PRIME_OPERANDS);
}
__device__ __forceinline__ void Loop<false, true>::tile(CUASR_MFMA64_TILE_ARGS) {
  unsigned m0_save;
  asm volatile(
#include "gen/mfma_asm_md_xk_tile.inc"
      CUASR_MFMA64_TILE_OPERANDS);
}
__device__ __forceinline__ void Loop<true, true>::prime(Regs &r, unsigned a_addr, unsigned b_addr) {
  asm volatile(
#include "gen/mfma_asm_md_kk_prime.inc"
      CUASR_MFMA64_PRIME_OPERANDS);
}
__device__ __forceinline__ void Loop<true, true>::tile(CUASR_MFMA64_TILE_ARGS) {
  unsigned m0_save;
  asm volatile(
#include "gen/mfma_asm_md_kk_tile.inc"
      CUASR_MFMA64_TILE_OPERANDS);
}

template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_mfma_direct_f64_kernel(Problem p) {
  __shared__ Smem sm;
  select_batch<double>(p);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;

  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const int ntiles = max(ke - kb, 0) / BK;  // the host sends only k ranges that are multiples of BK

  Regs r;
#pragma unroll
  for (int v = 0; v < 8; ++v) r.acc[v] = asm_d8(0.0);
#pragma unroll
  for (int v = 0; v < 4; ++v) r.frag[v] = asm_v16(0.0f);

  if (ntiles > 0) {
    const char *base_a = reinterpret_cast<const char *>(reinterpret_cast<const double *>(p.A) + (long long)m0 * p.sa_m + (long long)kb * p.sa_k);
    const char *base_b = reinterpret_cast<const char *>(reinterpret_cast<const double *>(p.B) + (long long)n0 * p.sb_n + (long long)kb * p.sb_k);
    const long long a_next = (long long)BK * p.sa_k * 8, b_next = (long long)BK * p.sb_k * 8;
    // this wave's pieces: 4 of the 16 of each panel
    unsigned off[8];
#pragma unroll
    for (int h = 0; h < 4; ++h) off[h] = lane_offset<A_KC, BM>((wave * 4 + h) * 64 + lane, p.sa_m, (unsigned)p.sa_k * 8u, m0, p.m);
#pragma unroll
    for (int h = 0; h < 4; ++h) off[4 + h] = lane_offset<B_KC, BN>((wave * 4 + h) * 64 + lane, p.sb_n, (unsigned)p.sb_k * 8u, n0, p.n);
    auto fetch = [&](int stage) {
#pragma unroll
      for (int h = 0; h < 4; ++h) dma16(base_a + off[h], &sm.a[stage][(wave * 4 + h) * 128]);
#pragma unroll
      for (int h = 0; h < 4; ++h) dma16(base_b + off[4 + h], &sm.b[stage][(wave * 4 + h) * 128]);
      base_a += a_next;
      base_b += b_next;
    };
    fetch(0);
    __syncthreads();  // waits for the loads first
    if (ntiles > 1) fetch(1);
    else {
      base_a += a_next;
      base_b += b_next;
    }
    // from here base_a / base_b point at tile 2

    // lane's LDS byte address of its operand for (stage 0, period 0, step 0, block 0): lane group g = lane / 16
    // takes the period's k-pair g
    const int g = lane >> 4, l16 = lane & 15;
    const unsigned a_base = (unsigned)(size_t)(__attribute__((address_space(3))) double *)&sm.a[0][0];
    const unsigned b_base = (unsigned)(size_t)(__attribute__((address_space(3))) double *)&sm.b[0][0];
    unsigned a_addr = a_base + (A_KC ? (g * BM + wm * 64 + l16) * 16 : (2 * g * BM + wm * 64 + l16) * 8);
    unsigned b_addr = b_base + (B_KC ? (g * BN + wn * 64 + l16) * 16 : (2 * g * BN + wn * 64 + l16) * 8);
    const unsigned m0_a0 = __builtin_amdgcn_readfirstlane(a_base + (wave * 4) * 1024);
    const unsigned m0_b0 = __builtin_amdgcn_readfirstlane(b_base + (wave * 4) * 1024);
    typedef Loop<A_KC, B_KC> L;
    L::prime(r, a_addr, b_addr);
    int stage = 0;
    for (int t = 0; t < ntiles; ++t) {
      // tile t sits in stage t % 2, which also takes tile t + 2 once this tile's barrier has passed
      L::tile(r, a_addr, b_addr, stage ? 0u - A_STAGE : A_STAGE, stage ? 0u - B_STAGE : B_STAGE, ntiles - (t + 2),
              m0_a0 + stage * A_STAGE, m0_b0 + stage * B_STAGE, off, base_a, base_b);
      base_a += a_next;
      base_b += b_next;
      stage ^= 1;
    }
    // the compiler does not see the matrix instructions inside the statements, so it cannot know that the
    // accumulators it reads next may still be on their way: the last one written needs 18 wait states
    asm volatile("s_nop 15\ns_nop 7"
                 : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]),
                   "+{v[64:79]}"(r.acc[4]), "+{v[80:95]}"(r.acc[5]), "+{v[96:111]}"(r.acc[6]), "+{v[112:127]}"(r.acc[7]));
  }

  // ---- epilogue.  Block (bi, bj), double e of lane l holds row l / 16 + 4 e, column l % 16 of the 16 x 16 block.
  double *out;
  long long ld_out;
  const bool partial = p.workspace != nullptr;
  double alpha = 1.0, beta = 0.0;
  bool source_needed = false;
  if (partial) {
    out = reinterpret_cast<double *>(p.workspace) + (long long)blockIdx.y * p.m * p.n;
    ld_out = p.n;
  } else {
    out = reinterpret_cast<double *>(p.D);
    ld_out = p.ldd;
    const EpilogueScalars<double> e = resolve_scalars<double>(p, kMultiplies);
    alpha = e.alpha;
    beta = e.beta;
    source_needed = e.source_needed;
  }
  const double *C = reinterpret_cast<const double *>(p.C);
  // A store instruction writes 128 consecutive bytes of four rows.  The four blocks of a block row are stored
  // register by register, so that four consecutive instructions write 512 consecutive bytes of each of their rows,
  // and a block row's source elements are requested together before any of its results is stored (D may be C, so
  // the compiler cannot move a load of C above a store to D by itself); one copy of the stores per case.
  const int col0 = n0 + wn * 64 + (lane & 15);
  auto store_all = [&](auto scaled, auto with_source) {
    constexpr bool SCALED = decltype(scaled)::value, SRC = decltype(with_source)::value;
#pragma unroll
    for (int bi = 0; bi < 4; ++bi) {
      double src[4][4];
      if constexpr (SRC) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int bj = 0; bj < 4; ++bj) {
            const int row = m0 + wm * 64 + bi * 16 + (lane >> 4) + 4 * e, col = col0 + bj * 16;
            if (row < p.m && col < p.n) src[e][bj] = C[(long long)row * p.ldc + col];
          }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int bj = 0; bj < 4; ++bj) {
          const int blk = 4 * bi + bj;
          const int row = m0 + wm * 64 + bi * 16 + (lane >> 4) + 4 * e, col = col0 + bj * 16;
          if (row < p.m && col < p.n) {
            double v = r.acc[blk >> 1][(blk & 1) * 4 + e];
            if constexpr (SCALED) v = alpha * v;
            if constexpr (SRC) v = v + beta * src[e][bj];
            out[(long long)row * ld_out + col] = v;
          }
        }
    }
  };
  if (partial) store_all(std::false_type{}, std::false_type{});
  else if (source_needed) store_all(std::true_type{}, std::true_type{});
  else store_all(std::true_type{}, std::false_type{});
}

// 16-byte vectors along the contiguous direction of either operand, whole k-tiles, every byte offset inside a
// tile in 32 bits
static bool can_run(const Problem &p) {
  auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;
  if (!al(p.A) || !al(p.B)) return false;
  if (a_xc ? (p.m % 2 || p.sa_k % 2) : (p.sa_k != 1 || p.sa_m % 2)) return false;
  if (b_xc ? (p.n % 2 || p.sb_k % 2) : (p.sb_k != 1 || p.sb_n % 2)) return false;
  if (p.k % BK) return false;
  if (p.workspace && p.k_per_slice % BK) return false;
  if (p.batch > 1 && (p.workspace || p.batch_a % 2 || p.batch_b % 2)) return false;  // every product 16-byte aligned
  const long long lim = 1LL << 29;  // elements
  if (p.sa_m * (long long)BM >= lim || p.sa_k * (long long)BK >= lim || p.sb_n * (long long)BN >= lim || p.sb_k * (long long)BK >= lim)
    return false;
  return true;
}

static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!can_run(p)) return hipErrorNotSupported;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN), slices = p.workspace ? p.slices : 1;
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  const bool a_kc = p.sa_m != 1, b_kc = p.sb_n != 1;
  auto go = [&](auto kernel) {
    launch_kernel(kernel, dim3((unsigned)tiles, (unsigned)slices, (unsigned)(p.batch > 1 ? p.batch : 1)), dim3(256), 0, s, p);
    return take_launch_status();
  };
  if (a_kc) return b_kc ? go(gemm_mfma_direct_f64_kernel<true, true>) : go(gemm_mfma_direct_f64_kernel<true, false>);
  return b_kc ? go(gemm_mfma_direct_f64_kernel<false, true>) : go(gemm_mfma_direct_f64_kernel<false, false>);
}

}  // namespace gemm_mfma_direct_f64

bool mfma_direct_f64_can_run(const Problem &p) { return gemm_mfma_direct_f64::can_run(p); }
hipError_t mfma_direct_f64_launch(const Problem &p, hipStream_t s) { return gemm_mfma_direct_f64::launch(p, s); }

}  // namespace cuasr_amd
