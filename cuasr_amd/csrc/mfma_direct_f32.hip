// plus-times for float on the matrix cores, hand-scheduled:
//     D = alpha * (A . B) + beta * C      with v_mfma_f32_32x32x2_f32
//
// The fast form of mfma_gemm_f32.hip (same instruction, same output tiles 128 x 256 and 128 x 128, same accumulator
// layout, same place in the library: the reference's SIMT kernel include/cuasr/gemm/kernel/srgemm.h:156-321
// for DefaultSemiRingConfiguration<plus, multiplies>) for products whose k range is a multiple of 16 and
// whose operands the direct-to-LDS loads can fetch (16-byte aligned rows).  What differs:
//   - panels go global -> LDS without passing registers (global_load_lds_dwordx4), three stages deep, the
//     tile two ahead requested at the top of each k-tile: 6 loads per wave and k-tile;
//   - the main loop is one generated asm statement per k-tile (gen_direct_asm.py, MfmaBody): 64 matrix
//     instructions, the LDS reads of the next 8 k issued right after the first 8 of them, one counted wait
//     and one barrier; nothing else.  The compiled loop carries ~40 address / wait / nop instructions per
//     k-quad that the matrix pipe has to wait for: 80.7 % MFMA busy there;
//   - a period of 8 k is walked as (k, k + 4), k = 0..3, so that a k-contiguous panel ([k/4][X][4] in
//     LDS, exactly the image the loads produce) feeds a 32-row block's four steps with ONE 16-byte read.
// The sum over k is formed in the instruction's order, so results agree with the host reference to
// rounding (|d - r| <= 1e-5 * sum_k |a||b|), like the compiled form.
#include "mfma_common.h"

namespace cuasr_amd {
namespace gemm_mfma_direct {

using mfma_panel::tile_coords;

constexpr int BM = 128, BK = 16, STAGES = 3;
constexpr unsigned A_STAGE = BK * BM * 4;

// NBN: 32-column blocks per wave.  4: output tile 128 x 256, waves of 64 x 128 (128 accumulator registers);
// 2: output tile 128 x 128, waves of 64 x 64 (64), for outputs whose wide tiles would leave most of a round of
// workgroups empty.
template <int NBN> struct Smem {
  float a[STAGES][BK * BM];
  float b[STAGES][BK * 64 * NBN];
};

typedef float asm_v16 __attribute__((ext_vector_type(16)));
template <int NBN> struct Regs {
  asm_v16 acc[2 * NBN];   // block (bm, bn) = acc[NBN bm + bn], from v0 up
  asm_v16 frag[1 + NBN / 2];  // A: v128 .. v143, B: v144 .. v143 + 8 NBN
};

// The panel's LDS image has X * 4 positions of 16 bytes; a wave's load fills 64 consecutive ones.
//   k-contiguous: position = quad * X + x     (4 consecutive k of one x)
//   x-contiguous: position = k * (X / 4) + x4 (4 consecutive x at one k)
// x is clamped to the matrix edge: what clamped positions fetch is never stored.
template <bool KC, int X> __device__ __forceinline__ unsigned lane_offset(int pos, long long s_x, unsigned s_k_bytes, int x0, int x_end) {
  if constexpr (KC) return (unsigned)(min(x0 + (pos % X), x_end - 1) - x0) * (unsigned)s_x * 4u + (unsigned)(pos / X) * 16u;
  else return (unsigned)(min(x0 + (pos % (X / 4)) * 4, x_end - 4) - x0) * 4u + (unsigned)(pos / (X / 4)) * s_k_bytes;
}

__device__ __forceinline__ void dma16(const char *src, float *lds_wave_base) {
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                   (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
}

// prime: the fragments of the first 8 k into their registers; the tile must have landed in LDS stage 0.
// tile: one k-tile of 16 -- 16 NBN matrix instructions per wave, the fetch of the tile two ahead (if fetch > 0), the
// workgroup barrier that hands the LDS stage back, and the fragments of the next tile's first 8 k.
template <bool A_KC, bool B_KC, int NBN> struct Loop;

#define CUASR_MFMA_TILE_ARGS(NBN)                                                                                             \
  Regs<NBN> &r, unsigned &a_addr, unsigned &b_addr, unsigned a_step, unsigned b_step, int fetch, unsigned m0_a,               \
      unsigned m0_b, const unsigned (&off)[2 + NBN], const char *base_a, const char *base_b
#define CUASR_MFMA_TAIL_OPERANDS                                                                                              \
          [a_addr] "+v"(a_addr), [b_addr] "+v"(b_addr), [m0_save] "=&s"(m0_save)                                              \
        : [a_step] "s"(a_step), [b_step] "s"(b_step), [fetch] "s"(fetch), [m0_a] "s"(m0_a), [m0_b] "s"(m0_b),                 \
          [off_a0] "v"(off[0]), [off_a1] "v"(off[1]), [off_b0] "v"(off[2]), [off_b1] "v"(off[3]),

#define CUASR_MFMA_PRIME4                                                                                                     \
        : "+{v[128:143]}"(r.frag[0]), "+{v[144:159]}"(r.frag[1]), "+{v[160:175]}"(r.frag[2])                                  \
        : [a_addr] "v"(a_addr), [b_addr] "v"(b_addr)                                                                          \
        : "memory"
#define CUASR_MFMA_PRIME2                                                                                                     \
        : "+{v[128:143]}"(r.frag[0]), "+{v[144:159]}"(r.frag[1])                                                              \
        : [a_addr] "v"(a_addr), [b_addr] "v"(b_addr)                                                                          \
        : "memory"
#define CUASR_MFMA_TILE4                                                                                                      \
        : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]),                  \
          "+{v[64:79]}"(r.acc[4]), "+{v[80:95]}"(r.acc[5]), "+{v[96:111]}"(r.acc[6]), "+{v[112:127]}"(r.acc[7]),              \
          "+{v[128:143]}"(r.frag[0]), "+{v[144:159]}"(r.frag[1]), "+{v[160:175]}"(r.frag[2]),                                 \
          CUASR_MFMA_TAIL_OPERANDS                                                                                            \
          [off_b2] "v"(off[4]), [off_b3] "v"(off[5]), [base_a] "s"(base_a), [base_b] "s"(base_b)                              \
        : "scc", "memory"
#define CUASR_MFMA_TILE2                                                                                                      \
        : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]),                  \
          "+{v[128:143]}"(r.frag[0]), "+{v[144:159]}"(r.frag[1]),                                                             \
          CUASR_MFMA_TAIL_OPERANDS                                                                                            \
          [base_a] "s"(base_a), [base_b] "s"(base_b)                                                                          \
        : "scc", "memory"

template <> struct Loop<true, false, 4> {
  static __device__ __forceinline__ void prime(Regs<4> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m_kx_prime.inc"
        CUASR_MFMA_PRIME4);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(4)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m_kx_tile.inc"
        CUASR_MFMA_TILE4);
  }
};
template <> struct Loop<false, false, 4> {
  static __device__ __forceinline__ void prime(Regs<4> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m_xx_prime.inc"
        CUASR_MFMA_PRIME4);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(4)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m_xx_tile.inc"
        CUASR_MFMA_TILE4);
  }
};
template <> struct Loop<false, true, 4> {
  static __device__ __forceinline__ void prime(Regs<4> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m_xk_prime.inc"
        CUASR_MFMA_PRIME4);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(4)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m_xk_tile.inc"
        CUASR_MFMA_TILE4);
  }
};
template <> struct Loop<true, true, 4> {
  static __device__ __forceinline__ void prime(Regs<4> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m_kk_prime.inc"
        CUASR_MFMA_PRIME4);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(4)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m_kk_tile.inc"
        CUASR_MFMA_TILE4);
  }
};
template <> struct Loop<true, false, 2> {
  static __device__ __forceinline__ void prime(Regs<2> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m2_kx_prime.inc"
        CUASR_MFMA_PRIME2);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(2)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m2_kx_tile.inc"
        CUASR_MFMA_TILE2);
  }
};
template <> struct Loop<false, false, 2> {
  static __device__ __forceinline__ void prime(Regs<2> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m2_xx_prime.inc"
        CUASR_MFMA_PRIME2);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(2)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m2_xx_tile.inc"
        CUASR_MFMA_TILE2);
  }
};
template <> struct Loop<false, true, 2> {
  static __device__ __forceinline__ void prime(Regs<2> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m2_xk_prime.inc"
        CUASR_MFMA_PRIME2);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(2)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m2_xk_tile.inc"
        CUASR_MFMA_TILE2);
  }
};
template <> struct Loop<true, true, 2> {
  static __device__ __forceinline__ void prime(Regs<2> &r, unsigned a_addr, unsigned b_addr) {
    asm volatile(
#include "gen/mfma_asm_m2_kk_prime.inc"
        CUASR_MFMA_PRIME2);
  }
  static __device__ __forceinline__ void tile(CUASR_MFMA_TILE_ARGS(2)) {
    unsigned m0_save;
    asm volatile(
#include "gen/mfma_asm_m2_kk_tile.inc"
        CUASR_MFMA_TILE2);
  }
};

template <bool A_KC, bool B_KC, int NBN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, NBN == 4 ? 2 : 3))) void gemm_mfma_direct_kernel(Problem p) {
  constexpr int BN = 64 * NBN, WN = 32 * NBN;
  constexpr unsigned B_STAGE = BK * BN * 4;
  __shared__ Smem<NBN> sm;
  select_batch<float>(p);
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

  Regs<NBN> r;
#pragma unroll
  for (int v = 0; v < 2 * NBN; ++v) r.acc[v] = asm_v16(0.0f);
#pragma unroll
  for (int v = 0; v < 1 + NBN / 2; ++v) r.frag[v] = asm_v16(0.0f);

  if (ntiles > 0) {
    const char *base_a = reinterpret_cast<const char *>(reinterpret_cast<const float *>(p.A) + (long long)m0 * p.sa_m + (long long)kb * p.sa_k);
    const char *base_b = reinterpret_cast<const char *>(reinterpret_cast<const float *>(p.B) + (long long)n0 * p.sb_n + (long long)kb * p.sb_k);
    const long long a_next = (long long)BK * p.sa_k * 4, b_next = (long long)BK * p.sb_k * 4;
    // this wave's pieces: 2 of the 8 of the A panel, NBN of the 4 NBN of the B panel
    unsigned off[2 + NBN];
#pragma unroll
    for (int h = 0; h < 2; ++h) off[h] = lane_offset<A_KC, BM>((wave * 2 + h) * 64 + lane, p.sa_m, (unsigned)p.sa_k * 4u, m0, p.m);
#pragma unroll
    for (int h = 0; h < NBN; ++h) off[2 + h] = lane_offset<B_KC, BN>((wave * NBN + h) * 64 + lane, p.sb_n, (unsigned)p.sb_k * 4u, n0, p.n);
    auto fetch = [&](int stage) {
#pragma unroll
      for (int h = 0; h < 2; ++h) dma16(base_a + off[h], &sm.a[stage][(wave * 2 + h) * 256]);
#pragma unroll
      for (int h = 0; h < NBN; ++h) dma16(base_b + off[2 + h], &sm.b[stage][(wave * NBN + h) * 256]);
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

    // lane's LDS byte address of its operand for (stage 0, period 0, step 0, block 0): lanes 0..31 take the
    // period's first k-quad, lanes 32..63 the second
    const int half = lane >> 5, l32 = lane & 31;
    const unsigned a_base = (unsigned)(size_t)(__attribute__((address_space(3))) float *)&sm.a[0][0];
    const unsigned b_base = (unsigned)(size_t)(__attribute__((address_space(3))) float *)&sm.b[0][0];
    unsigned a_addr = a_base + (A_KC ? (half * BM + wm * 64 + l32) * 16 : (half * 4 * BM + wm * 64 + l32) * 4);
    unsigned b_addr = b_base + (B_KC ? (half * BN + wn * WN + l32) * 16 : (half * 4 * BN + wn * WN + l32) * 4);
    const unsigned m0_a0 = __builtin_amdgcn_readfirstlane(a_base + (wave * 2) * 1024);
    const unsigned m0_b0 = __builtin_amdgcn_readfirstlane(b_base + (wave * NBN) * 1024);
    typedef Loop<A_KC, B_KC, NBN> L;
    L::prime(r, a_addr, b_addr);
    int stage = 0;
    for (int t = 0; t < ntiles; ++t) {
      const int next = stage + 1 == STAGES ? 0 : stage + 1, stage2 = next + 1 == STAGES ? 0 : next + 1;
      L::tile(r, a_addr, b_addr, (unsigned)((next - stage) * (int)A_STAGE), (unsigned)((next - stage) * (int)B_STAGE),
              ntiles - (t + 2), m0_a0 + stage2 * A_STAGE, m0_b0 + stage2 * B_STAGE, off, base_a, base_b);
      base_a += a_next;
      base_b += b_next;
      stage = next;
    }
    // the compiler does not see the matrix instructions inside the statements, so it cannot know that the
    // accumulators it reads next may still be on their way: the last one written needs 18 wait states
    if constexpr (NBN == 4)
      asm volatile("s_nop 15\ns_nop 7"
                   : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]),
                     "+{v[64:79]}"(r.acc[4]), "+{v[80:95]}"(r.acc[5]), "+{v[96:111]}"(r.acc[6]), "+{v[112:127]}"(r.acc[7]));
    else
      asm volatile("s_nop 15\ns_nop 7"
                   : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]));
  }

  // ---- epilogue.  Block (bi, bj), register r of lane l holds
  // row = 8*(r/4) + 4*(l/32) + r%4, column = l%32 of the 32 x 32 block.
  float *out;
  long long ld_out;
  const bool partial = p.workspace != nullptr;
  float alpha = 1.f, beta = 0.f;
  bool source_needed = false;
  if (partial) {
    out = reinterpret_cast<float *>(p.workspace) + (long long)blockIdx.y * p.m * p.n;
    ld_out = p.n;
  } else {
    out = reinterpret_cast<float *>(p.D);
    ld_out = p.ldd;
    const EpilogueScalars<float> e = resolve_scalars<float>(p, kMultiplies);
    alpha = e.alpha;
    beta = e.beta;
    source_needed = e.source_needed;
  }
  const float *C = reinterpret_cast<const float *>(p.C);
  // A store instruction writes 128 consecutive bytes of two rows.  The blocks of a block row are stored register by
  // register, so that NBN consecutive instructions write 128 NBN consecutive bytes of each of their two rows, and a
  // block row's source elements are requested together before any of its results is stored (D may be C, so the
  // compiler cannot move a load of C above a store to D by itself); one copy of the stores per case.
  const int col0 = n0 + wn * WN + (lane & 31);
  auto store_all = [&](auto scaled, auto with_source) {
    constexpr bool SCALED = decltype(scaled)::value, SRC = decltype(with_source)::value;
#pragma unroll
    for (int bi = 0; bi < 2; ++bi) {
      auto row_of = [&](int e) { return m0 + wm * 64 + bi * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4); };
      float src[16][NBN];
      if constexpr (SRC) {
#pragma unroll
        for (int e = 0; e < 16; ++e)
#pragma unroll
          for (int bj = 0; bj < NBN; ++bj) {
            const int row = row_of(e), col = col0 + bj * 32;
            if (row < p.m && col < p.n) src[e][bj] = C[(long long)row * p.ldc + col];
          }
      }
#pragma unroll
      for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int bj = 0; bj < NBN; ++bj) {
          const int row = row_of(e), col = col0 + bj * 32;
          if (row < p.m && col < p.n) {
            float v = r.acc[NBN * bi + bj][e];
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

// on top of mfma_panel::can_run: whole k-tiles only, and every byte offset inside a tile in 32 bits
static bool can_run(const Problem &p) {
  if (!mfma_panel::can_run(p)) return false;
  if (p.k % BK) return false;
  if (p.workspace && p.k_per_slice % BK) return false;
  if (p.batch > 1 && (p.workspace || p.batch_a % 4 || p.batch_b % 4)) return false;  // every product 16-byte aligned
  const long long lim = 1LL << 30;  // elements
  if (p.sa_m * (long long)BM >= lim || p.sa_k * (long long)BK >= lim || p.sb_n * 256LL >= lim || p.sb_k * (long long)BK >= lim)
    return false;
  return true;
}

// wide: the 128 x 256 tile, else 128 x 128
static hipError_t launch(const Problem &p, bool wide, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!can_run(p)) return hipErrorNotSupported;
  const int bn = wide ? 256 : 128;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + bn - 1) / bn), slices = p.workspace ? p.slices : 1;
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  const bool a_kc = p.sa_m != 1, b_kc = p.sb_n != 1;
  auto go = [&](auto kernel) {
    launch_kernel(kernel, dim3((unsigned)tiles, (unsigned)slices, (unsigned)(p.batch > 1 ? p.batch : 1)), dim3(256), 0, s, p);
    return take_launch_status();
  };
  if (wide) {
    if (a_kc) return b_kc ? go(gemm_mfma_direct_kernel<true, true, 4>) : go(gemm_mfma_direct_kernel<true, false, 4>);
    return b_kc ? go(gemm_mfma_direct_kernel<false, true, 4>) : go(gemm_mfma_direct_kernel<false, false, 4>);
  }
  if (a_kc) return b_kc ? go(gemm_mfma_direct_kernel<true, true, 2>) : go(gemm_mfma_direct_kernel<true, false, 2>);
  return b_kc ? go(gemm_mfma_direct_kernel<false, true, 2>) : go(gemm_mfma_direct_kernel<false, false, 2>);
}

}  // namespace gemm_mfma_direct

bool mfma_direct_f32_can_run(const Problem &p) { return gemm_mfma_direct::can_run(p); }
hipError_t mfma_direct_f32_launch(const Problem &p, bool wide, hipStream_t s) { return gemm_mfma_direct::launch(p, wide, s); }

}  // namespace cuasr_amd
