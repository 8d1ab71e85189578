// Vector-ALU SRGEMM tile for 4-byte element types whose panels go from global
// memory straight into LDS (global_load_lds_dwordx4), no staging registers.
//
// Same role as valu_tile.h (the reference's mainloop,
// include/cuasr/gemm/threadblock/srmma_pipelined.h:153-288, and kernel body,
// include/cuasr/gemm/kernel/srgemm.h:156-321), built around what was measured
// on gfx950:
//   * the vector ALU reaches its full issue rate only with an even number of
//     waves per SIMD, 4 or more: the kernel is held to 128 VGPRs (16 waves per
//     CU), which leaves no room for staging or double-buffered fragments;
//   * so panels go global -> LDS directly, and every fragment register is
//     refilled for the next k-pair right after its last use (see kpair()),
//     which hides the LDS latency without a second set of registers;
//   * v_min3_f32 folds two sums per accumulator: 1.5 instructions per term.
//
//   workgroup TY x TX threads (default 32 x 16 = 8 wave64), output tile
//   8*TY x 8*TX (256 x 128), k-tile 16, thread (ty, tx) owns 8 x 8 accumulators.
//
// A direct-to-LDS load writes lane l's 16 bytes at (wave-uniform base) + 16*l,
// so the LDS image of a panel is the order in which lanes fetch it and nothing
// can be transposed on the way.  A panel therefore has one of two LDS forms,
// chosen by which direction is contiguous in memory (X = panel width):
//   x-contiguous (x = m for A, n for B):  [k][X]      -> fragment = one 16-byte
//       read of 4 consecutive x at one k; the thread owns x = (X/2)*h + 4*t + e
//   k-contiguous:                         [k/4][X][4] -> fragment = one 8-byte
//       read of 2 consecutive k at one x; the thread owns x = (X/8)*i + t
// (t = ty for A, tx for B).
//
// Needs 16-byte aligned, vector-sized operands (see direct_ok); everything
// else runs on valu_tile.h.
#pragma once
#include <utility>

#include "direct_asm.h"
#include "semiring.h"

namespace cuasr_amd {

// RELAXED = false: 4 waves per SIMD (128 registers), one fragment set refilled in place (see kpair).
// RELAXED = true:  2 waves per SIMD (256 registers), two fragment sets, two LDS stages of a deeper
//                  k-tile: half the barriers, no register spills, no counted waits inside a k-pair.
template <typename T, int ADD, int MUL, bool A_KC, bool B_KC, int TY, int TX, int BK_ = 16, bool RELAXED = false>
struct DirectTile {
  static_assert(sizeof(T) == 4, "4-byte element types only");
  static constexpr int BM = 8 * TY, BN = 8 * TX, BK = BK_, THREADS = TY * TX, WAVES = THREADS / 64;
  // 1 KiB wave-loads per k-tile each wave issues for the A and the B panel
  static constexpr int LA = BM * BK / 256 / WAVES, LB = BN * BK / 256 / WAVES;
  static_assert(LA >= 1 && LB >= 1 && LA * WAVES * 256 == BM * BK && LB * WAVES * 256 == BN * BK, "panel must split evenly over the waves");
  typedef T vec4 __attribute__((ext_vector_type(4)));
  typedef T vec2 __attribute__((ext_vector_type(2)));

  // LDS ring: three stages when two workgroups of that size still fit a CU
  // (160 KiB), else two.  With three, the panel for k-tile t+2 can be fetched
  // at any time during tile t; with two it has to wait for the barrier that
  // frees the stage.
#ifdef CUASR_AMD_DIRECT_STAGES
  static constexpr int STAGES = CUASR_AMD_DIRECT_STAGES;
#else
  static constexpr int STAGES = RELAXED ? 2 : (3 * (BM + BN) * BK * 4 * (1024 / THREADS) <= 160 * 1024) ? 3 : 2;
#endif
  // k-pairs between two of a wave's loads of the panel two tiles ahead
#ifdef CUASR_AMD_DIRECT_SPREAD
  static constexpr int SPREAD = CUASR_AMD_DIRECT_SPREAD;
#else
  static constexpr int SPREAD = (BK / 2 - 2) / (LA + LB - 1) > 0 ? (BK / 2 - 2) / (LA + LB - 1) : 1;
#endif
  static_assert(RELAXED || (LA + LB - 1) * SPREAD < BK / 2, "all loads of a panel must be issued within one k-tile");
  struct Smem {
    T a[STAGES][BK * BM];
    T b[STAGES][BK * BN];
  };

  // ---- global -> LDS.  The panel's LDS image has 512 positions of 16 bytes;
  // wave w fills positions (2w + h)*64 + lane, h = 0, 1.  A position's address
  // is  (uniform base of this k-tile) + (per-lane byte offset);  the offset
  // has a part that never changes (the x index, clamped to the matrix edge) and,
  // for x-contiguous panels, a part that depends on how many k the tile holds
  // (k clamped to the last valid one; what clamped positions fetch is never
  // used).  All offsets are 32-bit: the host checks that a tile spans < 4 GiB.
  template <bool KC, int X>
  static __device__ __forceinline__ unsigned x_offset(int pos, long long s_x, int x0, int x_end) {
    if constexpr (KC) return (unsigned)(min(x0 + (pos % X), x_end - 1) - x0) * (unsigned)s_x * 4u;
    else return (unsigned)(min(x0 + (pos % (X / 4)) * 4, x_end - 4) - x0) * 4u;
  }
  // byte offset of position pos in a tile that holds kcount (1..16) valid k
  template <bool KC, int X>
  static __device__ __forceinline__ unsigned tile_offset(int pos, unsigned xoff, unsigned s_k_bytes, int kcount) {
    if constexpr (KC) return xoff + (unsigned)min((pos / X) * 4, kcount - 4) * 4u;
    else return xoff + (unsigned)min(pos / (X / 4), kcount - 1) * s_k_bytes;
  }

  static __device__ __forceinline__ void dma16(const T *src, T *lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                     (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
  }

  // ---- LDS -> registers, main loop.  Fragments of one k-pair (k = 2*kp + s)
  // for the thread's 8 rows (or columns) x.  They are fetched in the smallest
  // group one LDS read yields, so that a group can be refilled for the next
  // k-pair as soon as its last use is over:
  //   k-contiguous panel: one 8-byte read = both k of one x   (8 groups of 1 x)
  //   x-contiguous panel: one 16-byte read = 4 x at one k     (2 groups of 4 x, 2 reads each)
  // The reads are issued as asm so that THIS code, not the compiler, decides
  // where they sit and how long they may stay in flight: LDS reads complete in
  // order, so "s_waitcnt lgkmcnt(N)" lets the N youngest stay outstanding.
  // The compiler does not know a read is in flight, so a fragment must not be
  // touched (not even copied) between its read and the wait that covers it:
  // fragments live in exactly the vector registers the reads write, and the
  // wait statement names them.
  template <bool KC, int DUMMY = 0> struct Frag;
  template <int DUMMY> struct Frag<true, DUMMY> {
    vec2 v[8];  // v[x] = (k = 2kp, k = 2kp + 1)
    __device__ __forceinline__ T get(int s, int x) const { return v[x][s]; }
  };
  template <int DUMMY> struct Frag<false, DUMMY> {
    vec4 v[2][2];  // v[s][h] = x 4h .. 4h+3 at k = 2kp + s
    __device__ __forceinline__ T get(int s, int x) const { return v[s][x >> 2][x & 3]; }
  };
  // `addr` is the lane's LDS byte address of (stage, k-pair 0, x 0)
  // XT = threads along the panel's x direction; the panel is 8*XT wide
  template <int XT, int KP, int X> static __device__ __forceinline__ void refill_one(Frag<true> &f, unsigned addr) {
    asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(f.v[X]) : "v"(addr), "n"(((KP >> 1) * 8 * XT + X * XT) * 16 + (KP & 1) * 8));
  }
  template <int XT, int KP, int H> static __device__ __forceinline__ void refill_half(Frag<true> &f, unsigned addr) {
    refill_one<XT, KP, H * 4 + 0>(f, addr);
    refill_one<XT, KP, H * 4 + 1>(f, addr);
    refill_one<XT, KP, H * 4 + 2>(f, addr);
    refill_one<XT, KP, H * 4 + 3>(f, addr);
  }
  template <int XT, int KP, int H> static __device__ __forceinline__ void refill_half(Frag<false> &f, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.v[0][H]) : "v"(addr), "n"(((2 * KP + 0) * 8 * XT + H * 4 * XT) * 4));
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f.v[1][H]) : "v"(addr), "n"(((2 * KP + 1) * 8 * XT + H * 4 * XT) * 4));
  }
  template <bool KC> static constexpr int reads_per_half() { return KC ? 4 : 2; }
  // wait until at most N LDS reads are in flight; the fragments named become valid
  template <int N, int X> static __device__ __forceinline__ void wait_one(Frag<true> &f) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(f.v[X]) : "n"(N));
  }
  template <int N, int H> static __device__ __forceinline__ void wait_half(Frag<true> &f) {
    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f.v[H * 4]), "+v"(f.v[H * 4 + 1]), "+v"(f.v[H * 4 + 2]), "+v"(f.v[H * 4 + 3]) : "n"(N));
  }
  template <int N, int H> static __device__ __forceinline__ void wait_half(Frag<false> &f) {
    asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(f.v[0][H]), "+v"(f.v[1][H]) : "n"(N));
  }

  // the same for a single k (ragged last k-tile)
  template <bool KC, int XT> static __device__ __forceinline__ void load_frag1(T (&f)[8], const T *panel, int kk, int t) {
    if constexpr (KC) {
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = panel[((kk >> 2) * 8 * XT + i * XT + t) * 4 + (kk & 3)];
    } else {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const vec4 v = *reinterpret_cast<const vec4 *>(panel + kk * 8 * XT + h * 4 * XT + t * 4);
#pragma unroll
        for (int e = 0; e < 4; ++e) f[h * 4 + e] = v[e];
      }
    }
  }
  // tile-local index of the thread's i-th row / column
  template <bool KC, int XT> static __device__ __forceinline__ int own(int i, int t) {
    return KC ? i * XT + t : (i >> 2) * 4 * XT + t * 4 + (i & 3);
  }

  // CUASR_AMD_TILE_ORDER (measurement only; see profiles/direct_srgemm_minplus_f32_apsp4096.md): 0 = the order
  // described here, 1 = plain row-major tiles with no regard for the XCDs, 2 = blocks of 4 tile rows instead of 8
#ifndef CUASR_AMD_TILE_ORDER
#define CUASR_AMD_TILE_ORDER 0
#endif
  static __device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int &bm, int &bn) {
    const int total = tiles_m * tiles_n;
    if (CUASR_AMD_TILE_ORDER == 1) {
      bm = id / tiles_n;
      bn = id % tiles_n;
      return;
    }
    // consecutive workgroup ids land on consecutive XCDs (8, one L2 each):
    // give every XCD one contiguous run of the tile order
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr int GROUP = CUASR_AMD_TILE_ORDER == 2 ? 4 : 8;
    const int width = GROUP * tiles_n;
    const int group = id / width, first = group * GROUP;
    const int gsz = min(tiles_m - first, GROUP);
    bm = first + (id % width) % gsz;
    bn = (id % width) / gsz;
  }

  typedef Frag<A_KC> FragA;
  typedef Frag<B_KC> FragB;

  // one row x 4 columns (J0 .. J0+3) of one k-pair
  template <int I, int J0> static __device__ __forceinline__ void row4(T (&acc)[8][8], const FragA &a, const FragB &b) {
#pragma unroll
    for (int j = J0; j < J0 + 4; ++j) {
      if constexpr (fused_bit_term<ADD, MUL, T>::value) {
        acc[I][j] = term<ADD, MUL>(term<ADD, MUL>(acc[I][j], a.get(0, I), b.get(0, j)), a.get(1, I), b.get(1, j));
      } else {
        const T t0 = Op<MUL>::apply(a.get(0, I), b.get(0, j)), t1 = Op<MUL>::apply(a.get(1, I), b.get(1, j));
        acc[I][j] = fold<ADD, MUL>(t1, fold<ADD, MUL>(t0, acc[I][j]));
      }
    }
    // pin the row: computed here, not later (arithmetic has no side effect, so
    // only naming it in a volatile statement keeps it from drifting)
    asm volatile("" : "+v"(acc[I][J0]), "+v"(acc[I][J0 + 1]), "+v"(acc[I][J0 + 2]), "+v"(acc[I][J0 + 3]));
    __builtin_amdgcn_sched_barrier(0);
  }

  // LDS reads in flight when a k-pair starts, oldest first:
  //   B half 0 | A groups in row order | B half 1          (all for this k-pair)
  // phase 1, row I needs B half 0 and A up to row I; phase 2 needs B half 1,
  // which by then is followed only by the next k-pair's B half 0.
  template <int I> static constexpr int younger_than_a_row() {
    constexpr int nb = reads_per_half<B_KC>();
    if (A_KC) return (7 - I) + nb;                       // one read per row
    return (I < 4 ? reads_per_half<false>() : 0) + nb;   // half 0 covers rows 0..3, half 1 rows 4..7
  }
  template <int I> static __device__ __forceinline__ void phase1_row(T (&acc)[8][8], FragA &a, FragB &b) {
    if constexpr (I == 0) wait_half<younger_than_a_row<0>(), 0>(b);
    if constexpr (A_KC) wait_one<younger_than_a_row<I>(), I>(a);
    else if constexpr ((I & 3) == 0) wait_half<younger_than_a_row<I>(), (I >> 2)>(a);
    row4<I, 0>(acc, a, b);
  }
  template <int KP, int I> static __device__ __forceinline__ void phase2_row(T (&acc)[8][8], FragA &a, FragB &b, unsigned na_addr) {
    constexpr int NKP = (KP + 1) % (BK / 2);
    if constexpr (I == 0) wait_half<reads_per_half<B_KC>(), 1>(b);
    row4<I, 4>(acc, a, b);
    if constexpr (A_KC) refill_one<TY, NKP, I>(a, na_addr);
    else if constexpr ((I & 3) == 3) refill_half<TY, NKP, (I >> 2)>(a, na_addr);
  }
  template <int KP, typename Hook>
  static __device__ __forceinline__ void kpair(T (&acc)[8][8], FragA &a, FragB &b, unsigned &a_addr, unsigned &b_addr,
                                               Hook &&hook) {
    constexpr int LASTKP = BK / 2 - 1;
    constexpr int NKP = (KP + 1) % (LASTKP + 1);
    phase1_row<0>(acc, a, b);
    phase1_row<1>(acc, a, b);
    phase1_row<2>(acc, a, b);
    phase1_row<3>(acc, a, b);
    phase1_row<4>(acc, a, b);
    phase1_row<5>(acc, a, b);
    phase1_row<6>(acc, a, b);
    phase1_row<7>(acc, a, b);
    if constexpr (KP == LASTKP) wait_half<0, 1>(b);  // every read of this stage has returned before it is handed back
    // global -> LDS traffic and, in the last k-pair, the barrier and the switch
    // of a_addr / b_addr to the next stage: from here on the refills come from there
    hook(std::integral_constant<int, KP>{}, a_addr, b_addr);
    refill_half<TX, NKP, 0>(b, b_addr);
    phase2_row<KP, 0>(acc, a, b, a_addr);
    phase2_row<KP, 1>(acc, a, b, a_addr);
    phase2_row<KP, 2>(acc, a, b, a_addr);
    phase2_row<KP, 3>(acc, a, b, a_addr);
    phase2_row<KP, 4>(acc, a, b, a_addr);
    phase2_row<KP, 5>(acc, a, b, a_addr);
    phase2_row<KP, 6>(acc, a, b, a_addr);
    phase2_row<KP, 7>(acc, a, b, a_addr);
    refill_half<TX, NKP, 1>(b, b_addr);
  }
  template <int... KP, typename Hook>
  static __device__ __forceinline__ void tile_body(std::integer_sequence<int, KP...>, T (&acc)[8][8], FragA &a, FragB &b,
                                                   unsigned &a_addr, unsigned &b_addr, Hook &&hook) {
    (kpair<KP>(acc, a, b, a_addr, b_addr, hook), ...);
  }

  // ---- RELAXED main loop: fragment set KP & 1 is computed on while set (KP + 1) & 1 is being read.
  template <int KP> static __device__ __forceinline__ void issue_pair(FragA &a, FragB &b, unsigned a_addr, unsigned b_addr) {
    refill_half<TY, KP, 0>(a, a_addr);
    refill_half<TY, KP, 1>(a, a_addr);
    refill_half<TX, KP, 0>(b, b_addr);
    refill_half<TX, KP, 1>(b, b_addr);
  }
  template <int N> static __device__ __forceinline__ void wait_pair(FragA &a, FragB &b) {
    wait_half<N, 0>(a);
    wait_half<N, 1>(a);
    wait_half<N, 0>(b);
    wait_half<N, 1>(b);
  }
  template <int KP> static __device__ __forceinline__ void relaxed_kpair(T (&acc)[8][8], FragA (&a)[2], FragB (&b)[2], unsigned a_addr, unsigned b_addr) {
    constexpr int CUR = KP & 1, NXT = CUR ^ 1;
    // (the counter has 4 bits: with 16 reads per k-pair the wait also covers the first of the new ones)
    constexpr int READS_ = 2 * reads_per_half<A_KC>() + 2 * reads_per_half<B_KC>(), READS = READS_ < 15 ? READS_ : 15;
    if constexpr (KP + 1 < BK / 2) {
      issue_pair<KP + 1>(a[NXT], b[NXT], a_addr, b_addr);
      wait_pair<READS>(a[CUR], b[CUR]);  // the reads just issued may stay in flight, everything older has landed
    } else {
      wait_pair<0>(a[CUR], b[CUR]);
    }
    row4<0, 0>(acc, a[CUR], b[CUR]); row4<0, 4>(acc, a[CUR], b[CUR]);
    row4<1, 0>(acc, a[CUR], b[CUR]); row4<1, 4>(acc, a[CUR], b[CUR]);
    row4<2, 0>(acc, a[CUR], b[CUR]); row4<2, 4>(acc, a[CUR], b[CUR]);
    row4<3, 0>(acc, a[CUR], b[CUR]); row4<3, 4>(acc, a[CUR], b[CUR]);
    row4<4, 0>(acc, a[CUR], b[CUR]); row4<4, 4>(acc, a[CUR], b[CUR]);
    row4<5, 0>(acc, a[CUR], b[CUR]); row4<5, 4>(acc, a[CUR], b[CUR]);
    row4<6, 0>(acc, a[CUR], b[CUR]); row4<6, 4>(acc, a[CUR], b[CUR]);
    row4<7, 0>(acc, a[CUR], b[CUR]); row4<7, 4>(acc, a[CUR], b[CUR]);
  }
  template <int... KP>
  static __device__ __forceinline__ void relaxed_tile(std::integer_sequence<int, KP...>, T (&acc)[8][8], FragA (&a)[2], FragB (&b)[2],
                                                     unsigned a_addr, unsigned b_addr) {
    issue_pair<0>(a[0], b[0], a_addr, b_addr);
    (relaxed_kpair<KP>(acc, a, b, a_addr, b_addr), ...);
  }

  // what a workgroup does with the accumulators of a segment (one output tile, a range of k)
  enum : int {
    kEpilogue = 0,    // the whole product: D = add(mult(alpha, acc), mult(beta, C)); or a split-K slice: raw partials to the workspace
    kFoldOwned = 1,   // D already holds mult(beta, C) (or the identity): D = add(acc, D); this workgroup alone works on the tile
    kFoldShared = 2   // the same, but other workgroups fold other ranges of k into the same tile: one atomic fold per element
  };

  static __device__ __forceinline__ void run(const Problem &p, Smem &sm) {
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    int bm, bn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
    int kb = 0, ke = p.k;
    if (p.workspace) {
      kb = blockIdx.y * p.k_per_slice;
      ke = min(p.k, kb + p.k_per_slice);
    }
    segment(p, sm, bm * BM, bn * BN, kb, ke, kEpilogue);
  }

  // add(v, *addr) into *addr, atomically at device scope and without waiting for an answer.  The adds of the
  // semirings that run in this form all have a native atomic: xor / or on words; minimum and maximum of
  // floats through the integer atomics (a float without sign bit orders like its bits as a signed integer, one
  // with sign bit the other way round like its bits as an unsigned integer, and every float of the second kind is
  // below every float of the first both as a number and as a signed integer / above as an unsigned one).
  static __device__ __forceinline__ void atomic_fold(T *addr, T v) {
    const int bits = __builtin_bit_cast(int, v);
    int *si = reinterpret_cast<int *>(addr);
    unsigned *ui = reinterpret_cast<unsigned *>(addr);
    if constexpr (ADD == kBitXor) {
      __hip_atomic_fetch_xor(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if constexpr (ADD == kBitOr) {
      __hip_atomic_fetch_or(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if constexpr (ADD == kMinimum && is_fp<T>::value) {
      if (bits >= 0) __hip_atomic_fetch_min(si, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_fetch_max(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else if constexpr (ADD == kMaximum && is_fp<T>::value) {
      if (bits >= 0) __hip_atomic_fetch_max(si, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_fetch_min(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      // any other add: a compare-and-swap loop (no semiring that is launched in this form gets here)
      unsigned old = __hip_atomic_load(ui, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      while (true) {
        const unsigned want = __builtin_bit_cast(unsigned, fold_epilogue<ADD, MUL>(v, __builtin_bit_cast(T, old)));
        if (want == old) break;
        if (__hip_atomic_compare_exchange_strong(ui, &old, want, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
      }
    }
  }

  static __device__ __forceinline__ void segment(const Problem &p, Smem &sm, const int m0, const int n0, const int kb, const int ke,
                                                 const int mode) {
    const int tid = threadIdx.x, tx = tid % TX, ty = tid / TX, lane = tid & 63, wave = tid >> 6;
    const T *A = reinterpret_cast<const T *>(p.A);
    const T *B = reinterpret_cast<const T *>(p.B);
    const T ident = scalar_as<T>(p.add_identity);

    // each wave moves 2 x 1 KiB of the A panel and 2 x 1 KiB of the B panel per k-tile
    const char *base_a = reinterpret_cast<const char *>(A + (long long)m0 * p.sa_m + (long long)kb * p.sa_k);
    const char *base_b = reinterpret_cast<const char *>(B + (long long)n0 * p.sb_n + (long long)kb * p.sb_k);
    const long long a_step = (long long)BK * p.sa_k * 4, b_step = (long long)BK * p.sb_k * 4;
    const unsigned a_kbytes = (unsigned)p.sa_k * 4u, b_kbytes = (unsigned)p.sb_k * 4u;
    unsigned xa[LA], xb[LB];
#pragma unroll
    for (int h = 0; h < LA; ++h) xa[h] = x_offset<A_KC, BM>((wave * LA + h) * 64 + lane, p.sa_m, m0, p.m);
#pragma unroll
    for (int h = 0; h < LB; ++h) xb[h] = x_offset<B_KC, BN>((wave * LB + h) * 64 + lane, p.sb_n, n0, p.n);
    // piece q of a k-tile's traffic for this wave: its LA loads of A, then its LB loads of B
    auto fetch_piece = [&](int q, int stage, int kcount) {
      if (q < LA) {
        const int pos = (wave * LA + q) * 64 + lane;
        dma16(reinterpret_cast<const T *>(base_a + tile_offset<A_KC, BM>(pos, xa[q < LA ? q : 0], a_kbytes, kcount)),
              &sm.a[stage][(wave * LA + q) * 256]);
      } else {
        const int h = q - LA, pos = (wave * LB + h) * 64 + lane;
        dma16(reinterpret_cast<const T *>(base_b + tile_offset<B_KC, BN>(pos, xb[h < LB ? h : 0], b_kbytes, kcount)),
              &sm.b[stage][(wave * LB + h) * 256]);
      }
    };

    T acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[i][j] = ident;

    const int nfull = (ke - kb) / BK, rem = (ke - kb) - nfull * BK;  // whole k-tiles, then one ragged tile
    // k in tile t: BK for whole tiles, rem for the ragged one after them, 0 past the end
    auto tile_k = [&](int t) { return t < nfull ? BK : (t == nfull ? rem : 0); };
    // k-tile t lives in LDS stage t % STAGES; base_a / base_b point at the tile being fetched
    auto fetch_whole = [&](int t) {
      const int kc = tile_k(t);
      if (kc > 0) {
#pragma unroll
        for (int q = 0; q < LA + LB; ++q) fetch_piece(q, t % STAGES, kc);
      }
      base_a += a_step;
      base_b += b_step;
    };
    fetch_whole(0);
    __syncthreads();
    fetch_whole(1);  // from here base_a / base_b point at tile 2

    // Software pipeline without spare registers: every fragment group is
    // refilled for the NEXT k-pair right after its last use in this one.
    //   phase 1: rows 0..7 x columns 0..3   then refill B columns 0..3
    //   phase 2: rows 0..7 x columns 4..7,  refilling A row by row (or 4 rows
    //            at a time) as rows finish, then refill B columns 4..7
    // so each LDS read is issued 50..100 vector instructions before its use.
    // The last k-pair of a tile takes its refills from the other LDS stage,
    // which is why the barrier sits in the middle of that k-pair.
    // lane's LDS byte address of (stage 0, k-pair 0, x 0) in each panel
    const unsigned a_addr0 = (unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.a[0][0] + ty * 16;
    const unsigned b_addr0 = (unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.b[0][0] + tx * 16;
    typedef typename AsmLoop<T, ADD, MUL, A_KC, B_KC>::type Loop;
    if constexpr (!RELAXED && !std::is_void<Loop>::value && TY == 32 && TX == 16 && BK == 16 && STAGES == 3) {
      // The hand-scheduled main loop (direct_asm.h): accumulators and fragments live in fixed registers,
      // one asm statement per k-tile.  It fetches whole tiles only; a ragged last tile is fetched here,
      // by the same route as in the prologue, two tiles ahead like every other.
      static_assert(LA == 2 && LB == 1, "the generated loop moves two pieces of A and one of B per wave");
      if (nfull > 0) {
        AsmRegs r;
        const float ident_bits = __builtin_bit_cast(float, ident);
#pragma unroll
        for (int v = 0; v < 4; ++v)
#pragma unroll
          for (int e = 0; e < 16; ++e) r.acc[v][e] = ident_bits;
#pragma unroll
        for (int v = 0; v < 3; ++v) r.frag[v] = asm_v16(0.0f);
        // lane's global byte offsets inside a whole k-tile (the x clamp is part of xa / xb)
        const unsigned off_a0 = tile_offset<A_KC, BM>((wave * LA + 0) * 64 + lane, xa[0], a_kbytes, BK);
        const unsigned off_a1 = tile_offset<A_KC, BM>((wave * LA + 1) * 64 + lane, xa[1], a_kbytes, BK);
        const unsigned off_b0 = tile_offset<B_KC, BN>((wave * LB + 0) * 64 + lane, xb[0], b_kbytes, BK);
        // LDS byte address of this wave's first piece of each panel in stage 0 (wave-uniform)
        const unsigned m0_a0 = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.a[0][(wave * LA) * 256]);
        const unsigned m0_b0 = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.b[0][(wave * LB) * 256]);
        constexpr unsigned A_STAGE = BK * BM * 4, B_STAGE = BK * BN * 4;
        unsigned a_addr = a_addr0, b_addr = b_addr0;
        Loop::prime(r, a_addr, b_addr);
        int stage = 0;
        for (int t = 0; t < nfull; ++t) {
          const int next = stage + 1 == STAGES ? 0 : stage + 1, stage2 = next + 1 == STAGES ? 0 : next + 1;
          if (t + 2 == nfull && rem > 0) {
#pragma unroll
            for (int q = 0; q < LA + LB; ++q) fetch_piece(q, stage2, rem);
          }
          Loop::tile(r, a_addr, b_addr, (unsigned)((next - stage) * (int)A_STAGE), (unsigned)((next - stage) * (int)B_STAGE),
                     nfull - (t + 2), m0_a0 + stage2 * A_STAGE, m0_b0 + stage2 * B_STAGE, off_a0, off_a1, off_b0, base_a, base_b);
          base_a += a_step;
          base_b += b_step;
          stage = next;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            acc[i][j] = __builtin_bit_cast(T, (float)r.acc[i >> 1][(i & 1) * 8 + j]);
          }
      }
    } else if constexpr (RELAXED) {
      FragA a[2];
      FragB b[2];
      for (int t = 0; t < nfull; ++t) {
        const int stage = t & 1;
        relaxed_tile(std::make_integer_sequence<int, BK / 2>{}, acc, a, b, a_addr0 + stage * (BK * BM * 4),
                     b_addr0 + stage * (BK * BN * 4));
        __syncthreads();     // tile t+1 has landed (vmcnt waited first); nobody reads this stage any more
        fetch_whole(t + 2);  // ... so tile t+2 may overwrite it
      }
    } else {
    FragA a;
    FragB b;
    unsigned a_addr = a_addr0, b_addr = b_addr0;
    if (nfull > 0) {
      refill_half<TY, 0, 0>(a, a_addr);
      refill_half<TY, 0, 1>(a, a_addr);
      refill_half<TX, 0, 0>(b, b_addr);
      refill_half<TX, 0, 1>(b, b_addr);
      wait_half<0, 0>(a);
      wait_half<0, 1>(a);
      wait_half<0, 0>(b);
      wait_half<0, 1>(b);
    }
    int stage = 0;  // LDS stage of the tile being computed
    for (int t = 0; t < nfull; ++t) {
      const int next = stage + 1 == STAGES ? 0 : stage + 1;
      const int kc2 = tile_k(t + 2), stage2 = next + 1 == STAGES ? 0 : next + 1;  // tile t+2 and where it goes
      tile_body(std::make_integer_sequence<int, BK / 2>{}, acc, a, b, a_addr, b_addr, [&](auto kp, unsigned &aa, unsigned &ba) {
        constexpr int KP = decltype(kp)::value;
        // three stages: tile t+2's traffic is spread over the k-pairs of tile t, one load every
        // SPREAD k-pairs: a load's address registers are reloaded from scratch right before it, and
        // the wait for that reload also waits for the previous load, so the loads are kept apart
        if constexpr (STAGES == 3 && KP % SPREAD == 0 && KP / SPREAD < LA + LB) {
          if (kc2 > 0) fetch_piece(KP / SPREAD, stage2, kc2);
        }
        if constexpr (KP == BK / 2 - 1) {
          __syncthreads();  // tile t+1 has landed (vmcnt waited first); nobody reads this stage any more
          if constexpr (STAGES == 2) {  // two stages: only now is there room for tile t+2
            if (kc2 > 0) {
#pragma unroll
              for (int q = 0; q < LA + LB; ++q) fetch_piece(q, stage2, kc2);
            }
          }
          base_a += a_step;
          base_b += b_step;
          aa = a_addr0 + next * (BK * BM * 4);
          ba = b_addr0 + next * (BK * BN * 4);
        }
      });
      stage = next;
    }
    // The last k-pair has refilled the fragments for a k-pair that never runs.
    // Those reads must have returned before the compiler reuses the registers
    // for anything else (it cannot see that they are still being written).
    // Unconditional: with nothing pending the waits cost nothing, and a
    // path-insensitive check of the listing can then prove the drain.
    wait_half<0, 0>(a);
    wait_half<0, 1>(a);
    wait_half<0, 0>(b);
    wait_half<0, 1>(b);
    }  // !RELAXED
    const int buf = nfull % STAGES;
    if (rem > 0) {
      const T *pa = sm.a[buf], *pb = sm.b[buf];
#pragma unroll 1
      for (int kk = 0; kk < rem; ++kk) {
        T a[8], b[8];
        load_frag1<A_KC, TY>(a, pa, kk, ty);
        load_frag1<B_KC, TX>(b, pb, kk, tx);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[i][j] = term<ADD, MUL>(acc[i][j], a[i], b[j]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }

    if (mode != kEpilogue) {
      // ---- fold into D, which already holds the source term (alpha is the multiplicative identity here)
      T *D = reinterpret_cast<T *>(p.D);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row = m0 + own<A_KC, TY>(i, ty);
        if ((unsigned)row < (unsigned)p.m) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int col = n0 + own<B_KC, TX>(j, tx);
            if ((unsigned)col < (unsigned)p.n) {
              T *at = D + (long long)row * p.ldd + col;
              if (mode == kFoldShared) atomic_fold(at, acc[i][j]);
              else *at = fold_epilogue<ADD, MUL>(acc[i][j], *at);
            }
          }
        }
      }
      return;
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
      const int row = m0 + own<A_KC, TY>(i, ty);
      if ((unsigned)row < (unsigned)p.m) {  // unsigned: an index that is not one cannot pass
        if constexpr (!B_KC) {
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            const int col = n0 + g * 4 * TX + tx * 4;
            if ((unsigned)col < (unsigned)p.n) {  // n is a multiple of 4 here: the whole group is inside
              vec4 v;
#pragma unroll
              for (int c = 0; c < 4; ++c) v[c] = acc[i][g * 4 + c];
              if (!partial) {
#pragma unroll
                for (int c = 0; c < 4; ++c) v[c] = Op<MUL>::apply(e.alpha, v[c]);
                if (e.source_needed) {
                  const vec4 s = *reinterpret_cast<const vec4 *>(C + (long long)row * p.ldc + col);
#pragma unroll
                  for (int c = 0; c < 4; ++c) v[c] = fold_epilogue<ADD, MUL>(v[c], Op<MUL>::apply(e.beta, s[c]));
                }
              }
              *reinterpret_cast<vec4 *>(out + (long long)row * ld_out + col) = v;
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int col = n0 + own<true, TX>(j, tx);
            if ((unsigned)col < (unsigned)p.n) {
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

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC, int TY, int TX>
__global__ __launch_bounds__(TY *TX) __attribute__((amdgpu_waves_per_eu(4, 4))) void direct_srgemm_kernel(Problem p) {
  using Tile = DirectTile<T, ADD, MUL, A_KC, B_KC, TY, TX>;
  __shared__ typename Tile::Smem sm;
  select_batch<T>(p);
  Tile::run(p, sm);
}

// The same tile with the work of the last, partly filled round shared out evenly ("stream-K").  With G
// workgroups (two per compute unit) and T output tiles, the first floor(T / G) * G tiles are whole tiles as in
// the plain kernel, workgroup w taking tiles w, w + G, ...; the remaining R < G tiles are R x k-tiles units of work
// in tile-major order, of which workgroup w takes units [w * total / G, (w + 1) * total / G) -- a run of k-tiles
// that may end one output tile and begin the next.  For outputs whose tiles do not fill whole rounds of the chip
// (3072^2 is 288 tiles for 512 places, 5120^2 is 800) every workgroup then still has the same amount of work.
// The ranges of k of a shared tile meet in D: a launch before this one writes the source term into those tiles
// (prepare_fold_kernel), a workgroup that happens to have such a tile to itself folds its accumulators into it
// with plain loads and stores, the others with one atomic per element.  Only for adds whose result does not
// depend on the order or grouping of the terms, and with alpha = the multiplicative identity (so that nothing
// has to distribute over the add).
template <typename T, int ADD, int MUL, bool A_KC, bool B_KC, int TY, int TX>
__global__ __launch_bounds__(TY *TX) __attribute__((amdgpu_waves_per_eu(4, 4))) void direct_streamk_kernel(Problem p) {
  using Tile = DirectTile<T, ADD, MUL, A_KC, B_KC, TY, TX>;
  __shared__ typename Tile::Smem sm;
  const int tiles_m = (p.m + Tile::BM - 1) / Tile::BM, tiles_n = (p.n + Tile::BN - 1) / Tile::BN;
  const long long tiles = (long long)tiles_m * tiles_n, whole = tiles / gridDim.x * gridDim.x;
  bool first = true;
  int bm, bn;
  for (long long tile = blockIdx.x; tile < whole; tile += gridDim.x) {
    streamk_tile_coords(tile, tiles_m, tiles_n, bm, bn);
    if (!first) __syncthreads();  // every wave is done with the LDS panels of the previous tile
    first = false;
    Tile::segment(p, sm, bm * Tile::BM, bn * Tile::BN, 0, p.k, Tile::kEpilogue);
  }
  const long long ktiles = (p.k + Tile::BK - 1) / Tile::BK, total = (tiles - whole) * ktiles;
  long long u = total * blockIdx.x / gridDim.x;
  const long long end = total * (blockIdx.x + 1) / gridDim.x;
  while (u < end) {
    const long long r = u / ktiles;
    const int kt0 = (int)(u - r * ktiles), kt1 = (int)(end - r * ktiles < ktiles ? end - r * ktiles : ktiles);
    streamk_tile_coords(whole + r, tiles_m, tiles_n, bm, bn);
    if (!first) __syncthreads();
    first = false;
    Tile::segment(p, sm, bm * Tile::BM, bn * Tile::BN, kt0 * Tile::BK, min(p.k, kt1 * Tile::BK),
                  (kt0 == 0 && kt1 == ktiles) ? Tile::kFoldOwned : Tile::kFoldShared);
    u += kt1 - kt0;
  }
}

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void relaxed_srgemm_kernel(Problem p) {
  using Tile = DirectTile<T, ADD, MUL, A_KC, B_KC, 16, 16, 32, true>;
  __shared__ typename Tile::Smem sm;
  select_batch<T>(p);
  Tile::run(p, sm);
}

// can the direct tile run this (canonical) problem?
static inline bool direct_ok(const Problem &p) {
  auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  if (p.k <= 0 || !al(p.A) || !al(p.B)) return false;
  // every product of a batch in the grid starts at base + index * stride: the strides keep the 16-byte alignment
  if (p.batch > 1 && ((p.batch_a | p.batch_b | p.batch_c | p.batch_d) % 4)) return false;
  // 32-bit byte offsets inside one 128 x 16 tile
  const long long span = 4LL * 256 * (p.sa_m > p.sa_k ? p.sa_m : p.sa_k), span_b = 4LL * 256 * (p.sb_n > p.sb_k ? p.sb_n : p.sb_k);
  if (span >= (1LL << 31) || span_b >= (1LL << 31)) return false;
  if (a_kc ? (p.k % 4 || p.sa_m % 4) : (p.sa_m != 1 || p.m % 4 || p.sa_k % 4)) return false;
  if (b_kc ? (p.k % 4 || p.sb_n % 4) : (p.sb_n != 1 || p.n % 4 || p.sb_k % 4)) return false;
  if (!b_kc) {  // 16-byte stores of D (and loads of C)
    if (p.n % 4) return false;
    if (p.workspace) {
      if (!al(p.workspace)) return false;
    } else {
      if (!al(p.D) || p.ldd % 4) return false;
      if (p.C && (!al(p.C) || p.ldc % 4)) return false;
    }
  }
  return true;
}

// thread grid of the workgroup: 32 x 16 threads = 8 wave64, output tile 256 x 128
// (fastest of 16x16, 16x32, 32x16, 32x32 measured on MI355X at 4096^3)
#ifndef CUASR_AMD_DIRECT_TY
#define CUASR_AMD_DIRECT_TY 32
#define CUASR_AMD_DIRECT_TX 16
#endif

static inline bool direct_prefers_relaxed(const Problem &p) {
  return p.sa_k == 1 && p.sa_m != 1 && p.sb_k == 1 && p.sb_n != 1;
}

template <typename T, int ADD, int MUL> static hipError_t launch_relaxed(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!direct_ok(p)) return hipErrorNotSupported;
  const long long tiles = (long long)((p.m + 127) / 128) * ((p.n + 127) / 128);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1, p.batch);
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  if (a_kc && b_kc) launch_kernel((relaxed_srgemm_kernel<T, ADD, MUL, true, true>), grid, dim3(256), 0, s, p);
  else if (a_kc) launch_kernel((relaxed_srgemm_kernel<T, ADD, MUL, true, false>), grid, dim3(256), 0, s, p);
  else if (b_kc) launch_kernel((relaxed_srgemm_kernel<T, ADD, MUL, false, true>), grid, dim3(256), 0, s, p);
  else launch_kernel((relaxed_srgemm_kernel<T, ADD, MUL, false, false>), grid, dim3(256), 0, s, p);
  return take_launch_status();
}

template <typename T, int ADD, int MUL> static hipError_t launch_direct(const Problem &p, hipStream_t s) {
  // both operands k-contiguous: the 4-wave tile has to keep more lane addresses than it has
  // registers for and spills inside its main loop (58.7 vs 70.0 TOPS at 4096^3); the relaxed
  // tile does not.  Elsewhere the two are within noise of each other.
  if (direct_prefers_relaxed(p)) return launch_relaxed<T, ADD, MUL>(p, s);
  constexpr int TY = CUASR_AMD_DIRECT_TY, TX = CUASR_AMD_DIRECT_TX, BM = 8 * TY, BN = 8 * TX;
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!direct_ok(p)) return hipErrorNotSupported;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1, p.batch);
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  if (a_kc && b_kc) launch_kernel((direct_srgemm_kernel<T, ADD, MUL, true, true, TY, TX>), grid, dim3(TY * TX), 0, s, p);
  else if (a_kc) launch_kernel((direct_srgemm_kernel<T, ADD, MUL, true, false, TY, TX>), grid, dim3(TY * TX), 0, s, p);
  else if (b_kc) launch_kernel((direct_srgemm_kernel<T, ADD, MUL, false, true, TY, TX>), grid, dim3(TY * TX), 0, s, p);
  else launch_kernel((direct_srgemm_kernel<T, ADD, MUL, false, false, TY, TX>), grid, dim3(TY * TX), 0, s, p);
  return take_launch_status();
}

// stream-K form of the direct tile (see direct_streamk_kernel); `groups` workgroups, normally two per compute unit.
// The tiles from floor(tiles / groups) * groups on must already hold the source term (prepare_fold_kernel with this
// tile's extents, CUASR_AMD_DIRECT_TY * 8 x CUASR_AMD_DIRECT_TX * 8).
template <typename T, int ADD, int MUL> static hipError_t launch_direct_streamk(const Problem &p, int groups, hipStream_t s) {
  constexpr int TY = CUASR_AMD_DIRECT_TY, TX = CUASR_AMD_DIRECT_TX;
  if (p.m == 0 || p.n == 0 || p.k == 0) return hipSuccess;
  if (!direct_ok(p) || direct_prefers_relaxed(p) || p.workspace || p.batch != 1 || groups < 1) return hipErrorNotSupported;
  if constexpr (std::is_void<typename AsmLoop<T, ADD, MUL, false, false>::type>::value) {
    return hipErrorNotSupported;
  } else {
    const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
    dim3 grid((unsigned)groups);
    if (a_kc) launch_kernel((direct_streamk_kernel<T, ADD, MUL, true, false, TY, TX>), grid, dim3(TY * TX), 0, s, p);
    else if (b_kc) launch_kernel((direct_streamk_kernel<T, ADD, MUL, false, true, TY, TX>), grid, dim3(TY * TX), 0, s, p);
    else launch_kernel((direct_streamk_kernel<T, ADD, MUL, false, false, TY, TX>), grid, dim3(TY * TX), 0, s, p);
    return take_launch_status();
  }
}

}  // namespace cuasr_amd
