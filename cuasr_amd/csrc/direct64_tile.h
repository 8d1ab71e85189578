// Direct-to-LDS vector-ALU SRGEMM tile for 8-byte element types on gfx950.
//
// The fp64 counterpart of direct_tile.h's relaxed variant (same role in the
// reference: threadblock/srmma_pipelined.h:153-288, warp/srmma_simt.h:190-199,
// thread/srmma_sm50.h:118-146, kernel/srgemm.h:156-321).  fp64 vector
// instructions issue at 16 lanes per clock and there is no 3-input fp64
// min/max, so a term costs two instructions whatever the tile; what the tile
// can add is occupancy: the isolated 8x4 inner loop fed from LDS measures
// 28.4 TOPS at 2 waves per SIMD, 31.7 at 3 and 33.1 at 4.  The staged tile
// (valu_tile.h) needs ~216 registers for its staging registers, pointers and
// LDS store addresses and stays at 2 waves.  Here panels go global -> LDS
// without passing through registers, which leaves accumulators (64 registers),
// two fragment sets of one k-step (2 x 24) and a handful of addresses: 3 waves.
//
//   workgroup 256 threads (16 x 16), output tile 128 x 64, thread tile 8 x 4,
//   k-tile 16, two LDS stages (48 KiB; three workgroups per compute unit).
//
// LDS forms (the image equals the lane fetch order of the 16-byte loads):
//   x-contiguous operand: [k][X]       one 16-byte read = 2 x at one k
//   k-contiguous operand: [k/2][X][2]  one 8-byte read  = one x at one k
// Thread t of 16 along a panel owns, of its 8 (A) or 4 (B) rows/columns,
//   x-contiguous: pairs  x = (i/2)*32 + 2t + i%2      k-contiguous: x = 16 i + t.
// LDS reads are issued as asm with counted waits (see direct_tile.h for why):
// the set for k-step s+1 is read while step s is computed.
// Needs 16-byte aligned operands with even leading dimensions and extents
// (see direct64_ok); everything else goes to the staged tile.
#pragma once
#include <utility>
#include "semiring.h"

namespace cuasr_amd {

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC>
struct Direct64Tile {
  static_assert(sizeof(T) == 8, "8-byte element types only");
  static constexpr int BM = 128, BN = 64, BK = 16, WAVES = 4, STAGES = 2;
  // 1 KiB wave-loads per k-tile each wave issues for the A and the B panel
  static constexpr int LA = BM * BK * 8 / 1024 / WAVES, LB = BN * BK * 8 / 1024 / WAVES;  // 4, 2
  typedef T vec2 __attribute__((ext_vector_type(2)));

  struct Smem {
    T a[STAGES][BK * BM];
    T b[STAGES][BK * BN];
  };

  // ---- global -> LDS.  A panel's LDS image has X*BK/2 positions of 16 bytes; a position's
  // global address is (uniform base of this k-tile) + (per-lane byte offset, 32 bits: the host
  // checks that a tile spans less than 2 GiB).  Indices past the matrix edge or past the last
  // valid k of a ragged tile are clamped to the last valid vector (never used).
  template <bool KC, int X>
  static __device__ __forceinline__ unsigned tile_offset(int pos, long long s_x, unsigned s_k_bytes, int x0, int x_end, int kcount) {
    if constexpr (KC) {
      const int x = min(x0 + pos % X, x_end - 1) - x0, k = min((pos / X) * 2, kcount - 2);
      return (unsigned)x * (unsigned)s_x * 8u + (unsigned)k * 8u;
    } else {
      const int x = min(x0 + (pos % (X / 2)) * 2, x_end - 2) - x0, k = min(pos / (X / 2), kcount - 1);
      return (unsigned)x * 8u + (unsigned)k * s_k_bytes;
    }
  }
  static __device__ __forceinline__ void dma16(const char *src, T *lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                     (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
  }

  // ---- LDS -> registers: the fragments of one k-step.
  template <bool KC, int N, int DUMMY = 0> struct Frag;
  template <int N, int DUMMY> struct Frag<true, N, DUMMY> {
    T v[N];
    __device__ __forceinline__ T get(int i) const { return v[i]; }
  };
  template <int N, int DUMMY> struct Frag<false, N, DUMMY> {
    vec2 v[N / 2];
    __device__ __forceinline__ T get(int i) const { return v[i >> 1][i & 1]; }
  };
  typedef Frag<A_KC, 8> FragA;
  typedef Frag<B_KC, 4> FragB;
  template <bool KC, int N> static constexpr int reads() { return KC ? N : N / 2; }

  // `addr` is the lane's LDS byte address of (stage, k 0, its first x); X the panel width
  template <int X, int K, int I, int N> static __device__ __forceinline__ void read_one(Frag<true, N> &f, unsigned addr) {
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(f.v[I]) : "v"(addr), "n"(((K >> 1) * X + I * 16) * 16 + (K & 1) * 8));
  }
  template <int X, int K, int I, int N> static __device__ __forceinline__ void read_one(Frag<false, N> &f, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.v[I]) : "v"(addr), "n"((K * X + I * 32) * 8));
  }
  template <int X, int K, bool KC, int N, int... I>
  static __device__ __forceinline__ void read_all(Frag<KC, N> &f, unsigned addr, std::integer_sequence<int, I...>) {
    (read_one<X, K, I>(f, addr), ...);
  }
  template <int X, int K, bool KC, int N> static __device__ __forceinline__ void read_frag(Frag<KC, N> &f, unsigned addr) {
    read_all<X, K>(f, addr, std::make_integer_sequence<int, reads<KC, N>()>{});
  }
  // wait until at most CNT LDS reads are in flight; the fragments named become valid
  template <int CNT> static __device__ __forceinline__ void wait(Frag<true, 8> &f) {
    asm volatile("s_waitcnt lgkmcnt(%8)" : "+v"(f.v[0]), "+v"(f.v[1]), "+v"(f.v[2]), "+v"(f.v[3]), "+v"(f.v[4]), "+v"(f.v[5]), "+v"(f.v[6]), "+v"(f.v[7]) : "n"(CNT));
  }
  template <int CNT> static __device__ __forceinline__ void wait(Frag<false, 8> &f) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f.v[0]), "+v"(f.v[1]), "+v"(f.v[2]), "+v"(f.v[3]) : "n"(CNT));
  }
  template <int CNT> static __device__ __forceinline__ void wait(Frag<true, 4> &f) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f.v[0]), "+v"(f.v[1]), "+v"(f.v[2]), "+v"(f.v[3]) : "n"(CNT));
  }
  template <int CNT> static __device__ __forceinline__ void wait(Frag<false, 4> &f) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(f.v[0]), "+v"(f.v[1]) : "n"(CNT));
  }

  // tile-local index of the thread's i-th row / column
  template <bool KC> static __device__ __forceinline__ int own(int i, int t) {
    return KC ? i * 16 + t : (i >> 1) * 32 + t * 2 + (i & 1);
  }
  // the same fragments for a single k through ordinary loads (ragged last k-tile: nothing is in flight by then)
  template <bool KC, int N, int X> static __device__ __forceinline__ void load_frag1(T (&f)[N], const T *panel, int kk, int t) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int x = own<KC>(i, t);
      f[i] = KC ? panel[((kk >> 1) * X + x) * 2 + (kk & 1)] : panel[kk * X + x];
    }
  }

  static __device__ __forceinline__ void compute(T (&acc)[8][4], const FragA &a, const FragB &b) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = fold<ADD, MUL>(Op<MUL>::apply(a.get(i), b.get(j)), acc[i][j]);
      // pin the row: computed here, not later (only naming it in a volatile statement keeps it from drifting)
      asm volatile("" : "+v"(acc[i][0]), "+v"(acc[i][1]), "+v"(acc[i][2]), "+v"(acc[i][3]));
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  template <int K> static __device__ __forceinline__ void kstep(T (&acc)[8][4], FragA (&a)[2], FragB (&b)[2], unsigned a_addr, unsigned b_addr) {
    constexpr int CUR = K & 1, NXT = CUR ^ 1;
    constexpr int READS = reads<A_KC, 8>() + reads<B_KC, 4>();  // at most 12: fits the 4-bit counter
    if constexpr (K + 1 < BK) {
      read_frag<BM, K + 1>(a[NXT], a_addr);
      read_frag<BN, K + 1>(b[NXT], b_addr);
      wait<READS>(a[CUR]);  // the reads just issued may stay in flight, everything older has landed
      wait<READS>(b[CUR]);
    } else {
      wait<0>(a[CUR]);
      wait<0>(b[CUR]);
    }
    compute(acc, a[CUR], b[CUR]);
  }
  template <int... K>
  static __device__ __forceinline__ void whole_tile(std::integer_sequence<int, K...>, T (&acc)[8][4], FragA (&a)[2], FragB (&b)[2],
                                                   unsigned a_addr, unsigned b_addr) {
    read_frag<BM, 0>(a[0], a_addr);
    read_frag<BN, 0>(b[0], b_addr);
    (kstep<K>(acc, a, b, a_addr, b_addr), ...);
  }

  static __device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int &bm, int &bn) {
    const int total = tiles_m * tiles_n;
    // consecutive workgroup ids land on consecutive XCDs (8, one L2 each):
    // give every XCD one contiguous run of the tile order
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr int GROUP = 8;
    const int width = GROUP * tiles_n;
    const int group = id / width, first = group * GROUP;
    const int gsz = min(tiles_m - first, GROUP);
    bm = first + (id % width) % gsz;
    bn = (id % width) / gsz;
  }

  static __device__ __forceinline__ void run(const Problem &p, Smem &sm) {
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4, lane = tid & 63, wave = tid >> 6;
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    int bm, bn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
    const int m0 = bm * BM, n0 = bn * BN;
    const T *A = reinterpret_cast<const T *>(p.A);
    const T *B = reinterpret_cast<const T *>(p.B);
    const T ident = scalar_as<T>(p.add_identity);

    int kb = 0, ke = p.k;
    if (p.workspace) {
      kb = blockIdx.y * p.k_per_slice;
      ke = min(p.k, kb + p.k_per_slice);
    }

    const char *base_a = reinterpret_cast<const char *>(A + (long long)m0 * p.sa_m + (long long)kb * p.sa_k);
    const char *base_b = reinterpret_cast<const char *>(B + (long long)n0 * p.sb_n + (long long)kb * p.sb_k);
    const long long a_step = (long long)BK * p.sa_k * 8, b_step = (long long)BK * p.sb_k * 8;
    const unsigned a_kbytes = (unsigned)p.sa_k * 8u, b_kbytes = (unsigned)p.sb_k * 8u;
    // k-tile with kcount valid k into an LDS stage: each wave 4 x 1 KiB of A and 2 x 1 KiB of B
    auto fetch = [&](int stage, int kcount) {
      if (kcount > 0) {
#pragma unroll
        for (int q = 0; q < LA; ++q) {
          const int pos = (wave * LA + q) * 64 + lane;
          dma16(base_a + tile_offset<A_KC, BM>(pos, p.sa_m, a_kbytes, m0, p.m, kcount), &sm.a[stage][(wave * LA + q) * 128]);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q) {
          const int pos = (wave * LB + q) * 64 + lane;
          dma16(base_b + tile_offset<B_KC, BN>(pos, p.sb_n, b_kbytes, n0, p.n, kcount), &sm.b[stage][(wave * LB + q) * 128]);
        }
      }
      base_a += a_step;
      base_b += b_step;
    };

    T acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = ident;

    const int nfull = (ke - kb) / BK, rem = (ke - kb) - nfull * BK;  // whole k-tiles, then one ragged tile
    auto tile_k = [&](int t) { return t < nfull ? BK : (t == nfull ? rem : 0); };
    fetch(0, tile_k(0));
    __syncthreads();
    fetch(1, tile_k(1));

    // lane's LDS byte address of (stage 0, k 0, its first x) in each panel
    const unsigned a_addr0 = (unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.a[0][0] + ty * 16;
    const unsigned b_addr0 = (unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.b[0][0] + tx * 16;
    FragA a[2];
    FragB b[2];
    for (int t = 0; t < nfull; ++t) {
      const int stage = t & 1;
      whole_tile(std::make_integer_sequence<int, BK>{}, acc, a, b, a_addr0 + stage * (BK * BM * 8), b_addr0 + stage * (BK * BN * 8));
      __syncthreads();                 // tile t+1 has landed (vmcnt waited first); nobody reads this stage any more
      fetch(stage, tile_k(t + 2));     // ... so tile t+2 may overwrite it
    }
    if (rem > 0) {
      const int buf = nfull & 1;
      const T *pa = sm.a[buf], *pb = sm.b[buf];
#pragma unroll 1
      for (int kk = 0; kk < rem; ++kk) {
        T fa[8], fb[4];
        load_frag1<A_KC, 8, BM>(fa, pa, kk, ty);
        load_frag1<B_KC, 4, BN>(fb, pb, kk, tx);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = fold<ADD, MUL>(Op<MUL>::apply(fa[i], fb[j]), acc[i][j]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }

    // ---- epilogue: D = add(mult(alpha, acc), mult(beta, C)), or raw partials
    T *out;
    long long ld_out;
    const bool partial = p.workspace != nullptr;
    EpilogueScalars<T> e;
    if (partial) {
      out = reinterpret_cast<T *>(p.workspace) + (long long)blockIdx.y * p.m * p.n;
      ld_out = p.n;
      e.alpha = e.beta = e.ident = ident;
      e.source_needed = false;
    } else {
      out = reinterpret_cast<T *>(p.D);
      ld_out = p.ldd;
      e = resolve_scalars<T>(p, MUL);
    }
    const T *C = reinterpret_cast<const T *>(p.C);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = m0 + own<A_KC>(i, ty);
      if (row < p.m) {
        if constexpr (!B_KC) {
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            const int col = n0 + g * 32 + tx * 2;
            if (col < p.n) {  // n is even here: the pair is inside
              vec2 v = {acc[i][2 * g], acc[i][2 * g + 1]};
              if (!partial) {
#pragma unroll
                for (int c = 0; c < 2; ++c) v[c] = Op<MUL>::apply(e.alpha, v[c]);
                if (e.source_needed) {
                  const vec2 s = *reinterpret_cast<const vec2 *>(C + (long long)row * p.ldc + col);
#pragma unroll
                  for (int c = 0; c < 2; ++c) v[c] = fold_epilogue<ADD, MUL>(v[c], Op<MUL>::apply(e.beta, s[c]));
                }
              }
              *reinterpret_cast<vec2 *>(out + (long long)row * ld_out + col) = v;
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int col = n0 + own<true>(j, tx);
            if (col < p.n) {
              T v = acc[i][j];
              if (!partial) {
                v = Op<MUL>::apply(e.alpha, v);
                if (e.source_needed) v = fold_epilogue<ADD, MUL>(v, Op<MUL>::apply(e.beta, C[(long long)row * p.ldc + col]));
              }
              out[(long long)row * ld_out + col] = v;
            }
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

#ifndef CUASR_AMD_DIRECT64_WAVES
#define CUASR_AMD_DIRECT64_WAVES 3
#endif

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(CUASR_AMD_DIRECT64_WAVES, CUASR_AMD_DIRECT64_WAVES)))
void direct64_srgemm_kernel(Problem p) {
  using Tile = Direct64Tile<T, ADD, MUL, A_KC, B_KC>;
  __shared__ typename Tile::Smem sm;
  Tile::run(p, sm);
}

// can the fp64 direct tile run this (canonical) problem?
static inline bool direct64_ok(const Problem &p) {
  auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  if (p.k <= 0 || !al(p.A) || !al(p.B)) return false;
  // 32-bit byte offsets inside one tile
  const long long span = 8LL * 128 * (p.sa_m > p.sa_k ? p.sa_m : p.sa_k), span_b = 8LL * 128 * (p.sb_n > p.sb_k ? p.sb_n : p.sb_k);
  if (span >= (1LL << 31) || span_b >= (1LL << 31)) return false;
  if (a_kc ? (p.k % 2 || p.sa_m % 2) : (p.sa_m != 1 || p.m % 2 || p.sa_k % 2)) return false;
  if (b_kc ? (p.k % 2 || p.sb_n % 2) : (p.sb_n != 1 || p.n % 2 || p.sb_k % 2)) return false;
  if (!b_kc) {  // 16-byte stores of D (and loads of C)
    if (p.n % 2) return false;
    if (p.workspace) {
      if (!al(p.workspace)) return false;
    } else {
      if (!al(p.D) || p.ldd % 2) return false;
      if (p.C && (!al(p.C) || p.ldc % 2)) return false;
    }
  }
  return true;
}

template <typename T, int ADD, int MUL> static hipError_t launch_direct64(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!direct64_ok(p)) return hipErrorNotSupported;
  const long long tiles = (long long)((p.m + 127) / 128) * ((p.n + 63) / 64);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1);
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  if (a_kc && b_kc) hipLaunchKernelGGL((direct64_srgemm_kernel<T, ADD, MUL, true, true>), grid, dim3(256), 0, s, p);
  else if (a_kc) hipLaunchKernelGGL((direct64_srgemm_kernel<T, ADD, MUL, true, false>), grid, dim3(256), 0, s, p);
  else if (b_kc) hipLaunchKernelGGL((direct64_srgemm_kernel<T, ADD, MUL, false, true>), grid, dim3(256), 0, s, p);
  else hipLaunchKernelGGL((direct64_srgemm_kernel<T, ADD, MUL, false, false>), grid, dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace cuasr_amd
