// LDS-staged, register-blocked vector-ALU SRGEMM tile kernel for gfx950.
//
// Plays the role of the reference's threadblock/warp/thread hierarchy
// (include/cuasr/gemm/threadblock/srmma_pipelined.h:153-288,
//  include/cuasr/gemm/warp/srmma_simt.h:190-199,
//  include/cuasr/gemm/thread/srmma_sm50.h:118-146, include/cuasr/arch/srmma.h:84-91)
// and of the kernel body include/cuasr/gemm/kernel/srgemm.h:156-321, with a
// design of its own:
//   * one workgroup = 256 threads = 4 wave64, output tile (16*TM) x (16*TN);
//   * thread (ty, tx) of a 16x16 arrangement owns TM x TN accumulators in
//     16-byte groups, so every LDS fragment read is one ds_read_b128 and every
//     D access one 16-byte global access;
//   * A and B panels live in LDS k-major ([kk][m] and [kk][n]), double
//     buffered, one barrier per k-tile; the next tile's global loads are in
//     flight while the current tile is computed;
//   * A ragged last k-tile is handled by shortening the loop, never by padding
//     (a padded identity is not neutral for every semiring), so the result is
//     the host reference's for any K.
// blockIdx.x walks output tiles through an XCD-aware, row-grouped order;
// blockIdx.y is the split-K slice.
#pragma once
#include "semiring.h"

#ifndef WAVES_ATTR
#define WAVES_ATTR
#endif
namespace cuasr_amd {

// VEC: 16-byte global accesses.  CAREFUL (with VEC): operands of any extent, leading dimension and
// element alignment -- edge vectors and the last k-tile are treated separately (see Mover); without
// it the host guarantees extents along the contiguous directions that are multiples of the vector.
template <typename T, int ADD, int MUL, int TM, int TN, int BK, bool VEC, bool CAREFUL = false>
struct ValuTile {
  // k-steps taken together: two let a pair of sums meet in one 3-input min/max (4-byte types);
  // 8-byte types have no 3-input instructions, and one k-step per fragment set halves the
  // registers the fragments take
  static constexpr int KU = sizeof(T) == 8 ? 1 : 2;
  static constexpr int VW = 16 / sizeof(T);
  static constexpr int BM = 16 * TM, BN = 16 * TN;
  static constexpr int LDA = BM + VW, LDB = BN + VW;
  static constexpr int A_ELEMS = BM * BK / 256, B_ELEMS = BN * BK / 256;
  static constexpr int HM = TM / VW, GN = TN / VW;
  static_assert(A_ELEMS >= VW && B_ELEMS >= VW && HM >= 1 && GN >= 1, "tile too small");
  static_assert(BK % VW == 0 && BK % KU == 0, "BK must hold whole vectors");
  static_assert(A_ELEMS % VW == 0 && B_ELEMS % VW == 0 && A_ELEMS * 256 == BM * BK && B_ELEMS * 256 == BN * BK,
                "a panel must split into whole vectors per thread");
  typedef T vec_t __attribute__((ext_vector_type(VW)));
  // the same vector in global memory, where only element alignment is required (the hardware
  // takes 16-byte loads and stores at any 4-byte boundary)
  typedef T gvec_t __attribute__((ext_vector_type(VW), aligned(sizeof(T))));

  // Two semirings whose inner loop does not compute with the operators as written:
  //   MASKED     or-and.  `lhs && rhs`, `lhs || rhs` (functional.h:212, :252) only look at whether
  //              an operand is zero, so the panels go to LDS as 32-bit masks (all ones / zero)
  //              whatever the element type, a term is one three-input bit operation `acc | (a & b)`
  //              on 32-bit words, and the epilogue turns the mask back into the 1 / 0 the operators
  //              return.
  //   ZERO_SIGN  min-times / max-times on floating point.  The hardware min / max give the
  //              reference's value, but on a tie between +0 and -0 the reference keeps the newer
  //              product (host_srgemm.h:87 with functional.h:132, :172) and the hardware keeps -0.
  //              A zero result therefore has the sign of the LAST zero product of the k range,
  //              which the epilogue looks up for the accumulators that ended at zero.
  static constexpr bool MASKED = ADD == kLogicalOr && MUL == kLogicalAnd;
  static constexpr bool ZERO_SIGN = is_fp<T>::value && MUL == kMultiplies && (ADD == kMinimum || ADD == kMaximum);
  using S = typename std::conditional<MASKED, uint32_t, T>::type;  // what LDS, fragments and accumulators hold
  typedef S svec_t __attribute__((ext_vector_type(VW)));
  static __device__ __forceinline__ S staged(T x) {
    if constexpr (MASKED) return truth(x) ? 0xFFFFFFFFu : 0u;
    else return x;
  }
  static constexpr bool FUSED = fused_bit_term<ADD, MUL, T>::value;
  static __device__ __forceinline__ S term(S acc, S a, S b) {
    if constexpr (MASKED) return or_and_term(acc, a, b);
    else if constexpr (ZERO_SIGN) return Op<ADD>::apply(acc, Op<MUL>::apply(a, b));
    else return cuasr_amd::term<ADD, MUL>(acc, a, b);
  }
  // ZERO_SIGN: the last product of the k range that is zero (acc itself when there is none: an
  // empty range, or a zero identity).  Not inlined: it runs for the few accumulators that ended
  // at zero, after the main loop.
  static __device__ __attribute__((noinline)) T last_zero_product(const T *a_row, long long sa_k, const T *b_col,
                                                                 long long sb_k, int kcount, T acc) {
    for (int kk = kcount - 1; kk >= 0; --kk) {
      const T prod = a_row[(long long)kk * sa_k] * b_col[(long long)kk * sb_k];
      if (prod == T(0)) return prod;
    }
    return acc;
  }

  struct Smem {
    S a[2][BK][LDA];
    S b[2][BK][LDB];
  };

  // ---- global -> registers.  ROWS is the panel extent (BM or BN), s_x the
  // element stride along the panel's m/n index, s_k along k.  Indices that
  // fall outside the matrix are clamped to its last row/column/k: what is
  // fetched there is never used (rows and columns past the edge are not
  // stored, k past the end is not iterated), so no branch and no fill value.
  //   VEC:  a thread owns ELEMS/VW groups of VW elements consecutive along the
  //         panel's contiguous direction, one 16-byte load each; the host
  //         guarantees alignment and that extents along that direction are
  //         multiples of VW, so a clamped group never straddles the edge.
  //   !VEC: a thread owns ELEMS single elements.
  template <int ROWS, int ELEMS>
  static __device__ __forceinline__ void load_panel(T (&r)[ELEMS], const T *base, long long s_x, long long s_k,
                                                    int x0, int x_end, int k0, int k_end, bool x_contig) {
    const int tid = threadIdx.x & 255;
    if constexpr (VEC) {
      constexpr int VECS = ELEMS / VW, XV = ROWS / VW, KV = BK / VW;
#pragma unroll
      for (int p = 0; p < VECS; ++p) {
        const int v = tid + 256 * p;
        const int xx = min(x0 + (x_contig ? (v % XV) * VW : v / KV), x_end - (x_contig ? VW : 1));
        const int kk = min(k0 + (x_contig ? v / XV : (v % KV) * VW), k_end - (x_contig ? 1 : VW));
        const vec_t t = *reinterpret_cast<const vec_t *>(base + (long long)xx * s_x + (long long)kk * s_k);
#pragma unroll
        for (int e = 0; e < VW; ++e) r[p * VW + e] = t[e];
      }
    } else {
#pragma unroll
      for (int p = 0; p < ELEMS; ++p) {
        const int el = tid + 256 * p;
        const int xx = min(x0 + (x_contig ? el % ROWS : el / BK), x_end - 1);
        const int kk = min(k0 + (x_contig ? el / ROWS : el % BK), k_end - 1);
        r[p] = base[(long long)xx * s_x + (long long)kk * s_k];
      }
    }
  }

  // ---- the same ownership with the addressing done once (VEC only): a thread
  // keeps one pointer per 16-byte vector, at the vector's place in the first
  // k-tile, and moves it one k-tile along per iteration -- two integer
  // instructions per vector and tile instead of the index arithmetic of
  // load_panel.  Any extents, leading dimensions and (element) alignment:
  //   * a vector that lies wholly past the panel's edge points at the last
  //     whole vector inside the matrix (what it fetches is never used);
  //   * a vector that straddles the edge of an x-contiguous panel (extent not
  //     a multiple of VW) reads on into the padding or the next k row: valid
  //     memory of the same matrix as long as a later k row exists, which is
  //     why the LAST k-tile of a workgroup is never fetched this way but by
  //     load_last, element by element with both indices clamped.
  template <int ROWS, int ELEMS> struct Mover {
    static constexpr int VECS = ELEMS / VW, XV = ROWS / VW, KV = BK / VW;
    const T *src[VECS];
    long long step;
    __device__ __forceinline__ void init(const T *base, long long s_x, long long s_k, int x0, int x_end, int k0,
                                         bool x_contig) {
      const int tid = threadIdx.x & 255;
      step = (long long)BK * s_k;
#pragma unroll
      for (int p = 0; p < VECS; ++p) {
        const int v = tid + 256 * p;
        int xx = x0 + (x_contig ? (v % XV) * VW : v / KV);
        if (x_contig) xx = xx >= x_end ? x_end - VW : xx;
        else xx = min(xx, x_end - 1);
        const int kk = k0 + (x_contig ? v / XV : (v % KV) * VW);
        src[p] = base + (long long)xx * s_x + (long long)kk * s_k;
      }
    }
    __device__ __forceinline__ void load(T (&r)[ELEMS]) {
#pragma unroll
      for (int p = 0; p < VECS; ++p) {
        const gvec_t t = *reinterpret_cast<const gvec_t *>(src[p]);
#pragma unroll
        for (int e = 0; e < VW; ++e) r[p * VW + e] = t[e];
        src[p] += step;
      }
    }
    // !CAREFUL: ragged last k-tile; vectors past its end re-read its last valid vector
    __device__ __forceinline__ void load_ragged(T (&r)[ELEMS], long long s_k, int kcount, bool x_contig) {
      const int tid = threadIdx.x & 255;
#pragma unroll
      for (int p = 0; p < VECS; ++p) {
        const int v = tid + 256 * p;
        const int kl = x_contig ? v / XV : (v % KV) * VW;         // the vector's first k inside the tile
        const int back = max(kl - (kcount - (x_contig ? 1 : VW)), 0);  // steps of k past the last valid vector
        const gvec_t t = *reinterpret_cast<const gvec_t *>(src[p] - (long long)back * s_k);
#pragma unroll
        for (int e = 0; e < VW; ++e) r[p * VW + e] = t[e];
        src[p] += step;
      }
    }
  };

  // The last k-tile (k0 .. k_end, 1 .. BK values of k) of a panel, straight into its LDS stage:
  // every element with its own clamped indices.  Deliberately NOT inlined: it runs once per
  // workgroup, and inlined into the main loop its address arithmetic costs the loop 60-80
  // registers (a wave less per SIMD for the quarter-size tile).
  template <int ROWS, int LD>
  static __device__ __attribute__((noinline)) void fill_last(S (*dst)[LD], const T *base, long long s_x, long long s_k, int x0,
                                                             int x_end, int k0, int k_end, bool x_contig) {
    const int tid = threadIdx.x & 255;
    const int xmax = x_end - 1 - x0, kmax = k_end - 1 - k0;
    const T *tile = base + (long long)x0 * s_x + (long long)k0 * s_k;
    constexpr int N = ROWS * BK / 256;
    T r[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {  // all loads in flight together
      const int el = tid + 256 * i;
      const int x = x_contig ? el % ROWS : el / BK, kk = x_contig ? el / ROWS : el % BK;
      r[i] = tile[(long long)min(x, xmax) * s_x + (long long)min(kk, kmax) * s_k];
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int el = tid + 256 * i;
      dst[x_contig ? el / ROWS : el % BK][x_contig ? el % ROWS : el / BK] = staged(r[i]);
    }
  }

  // ---- registers -> LDS ([kk][x], k-major), same ownership as load_panel
  template <int ROWS, int LD, int ELEMS>
  static __device__ __forceinline__ void store_panel(const T (&r)[ELEMS], S (*dst)[LD], bool x_contig) {
    const int tid = threadIdx.x & 255;
    if constexpr (VEC) {
      constexpr int VECS = ELEMS / VW, XV = ROWS / VW, KV = BK / VW;
      if (x_contig) {
#pragma unroll
        for (int p = 0; p < VECS; ++p) {
          const int v = tid + 256 * p;
          svec_t t;
#pragma unroll
          for (int e = 0; e < VW; ++e) t[e] = staged(r[p * VW + e]);
          *reinterpret_cast<svec_t *>(&dst[v / XV][(v % XV) * VW]) = t;
        }
      } else {
#pragma unroll
        for (int p = 0; p < VECS; ++p) {
          const int v = tid + 256 * p;
#pragma unroll
          for (int e = 0; e < VW; ++e) dst[(v % KV) * VW + e][v / KV] = staged(r[p * VW + e]);
        }
      }
    } else {
#pragma unroll
      for (int p = 0; p < ELEMS; ++p) {
        const int el = tid + 256 * p;
        dst[x_contig ? el / ROWS : el % BK][x_contig ? el % ROWS : el / BK] = staged(r[p]);
      }
    }
  }

  static __device__ __forceinline__ void step(S (&acc)[TM][TN], const S (*as)[LDA], const S (*bs)[LDB], int kk,
                                              int ty, int tx) {
    S a[TM], b[TN];
#pragma unroll
    for (int h = 0; h < HM; ++h) {
      const svec_t t = *reinterpret_cast<const svec_t *>(&as[kk][ty * VW + h * 16 * VW]);
#pragma unroll
      for (int e = 0; e < VW; ++e) a[h * VW + e] = t[e];
    }
#pragma unroll
    for (int g = 0; g < GN; ++g) {
      const svec_t t = *reinterpret_cast<const svec_t *>(&bs[kk][tx * VW + g * 16 * VW]);
#pragma unroll
      for (int e = 0; e < VW; ++e) b[g * VW + e] = t[e];
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = term(acc[i][j], a[i], b[j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- whole k-tile, two k-steps at a time (per accumulator two products and
  // two adds, which the min/max semirings fold into one 3-input instruction;
  // the scheduling barrier after each row keeps the products of one row from
  // piling up across rows) and software pipelined: the fragments of k-pair
  // kp + 1 are read from LDS while k-pair kp is computed (two fragment sets in
  // registers), so a wave does not stall on LDS latency at every k-pair.
  // (integer element types keep the rolled loop: unrolled, their tiles take the
  // compiler ten minutes each, and they are not the throughput cases)
  static constexpr bool PIPELINED = T(0.5) != T(0);  // floating-point element type
  struct Frag2 {
    S a[KU][TM], b[KU][TN];
  };
  static __device__ __forceinline__ void load_frag2(Frag2 &f, const S (*as)[LDA], const S (*bs)[LDB], int kk, int ty, int tx) {
#pragma unroll
    for (int s = 0; s < KU; ++s) {
#pragma unroll
      for (int h = 0; h < HM; ++h) {
        const svec_t t = *reinterpret_cast<const svec_t *>(&as[kk + s][ty * VW + h * 16 * VW]);
#pragma unroll
        for (int e = 0; e < VW; ++e) f.a[s][h * VW + e] = t[e];
      }
#pragma unroll
      for (int g = 0; g < GN; ++g) {
        const svec_t t = *reinterpret_cast<const svec_t *>(&bs[kk + s][tx * VW + g * 16 * VW]);
#pragma unroll
        for (int e = 0; e < VW; ++e) f.b[s][g * VW + e] = t[e];
      }
    }
  }
  static __device__ __forceinline__ void compute2(S (&acc)[TM][TN], const Frag2 &f) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        if constexpr (MASKED || ZERO_SIGN || FUSED) {
          // (the bit terms are one opaque instruction each: written as `acc | (a & b)`, integer or
          // being associative, the compiler regroups the terms of a whole unrolled k-tile into a
          // tree and needs a register for every a & b of it)
#pragma unroll
          for (int s = 0; s < KU; ++s) acc[i][j] = term(acc[i][j], f.a[s][i], f.b[s][j]);
        } else if constexpr (KU == 2) {
          const T t0 = Op<MUL>::apply(f.a[0][i], f.b[0][j]), t1 = Op<MUL>::apply(f.a[1][i], f.b[1][j]);
          acc[i][j] = fold<ADD, MUL>(t1, fold<ADD, MUL>(t0, acc[i][j]));
        } else {
          acc[i][j] = fold<ADD, MUL>(Op<MUL>::apply(f.a[0][i], f.b[0][j]), acc[i][j]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  static __device__ __forceinline__ void whole_tile(S (&acc)[TM][TN], const S (*as)[LDA], const S (*bs)[LDB], int ty, int tx) {
    constexpr int STEPS = BK / KU;
    if constexpr (PIPELINED) {
      Frag2 f[2];
      load_frag2(f[0], as, bs, 0, ty, tx);
#pragma unroll
      for (int kp = 0; kp < STEPS; ++kp) {
        if (kp + 1 < STEPS) load_frag2(f[(kp + 1) & 1], as, bs, KU * (kp + 1), ty, tx);
        __builtin_amdgcn_sched_barrier(0);
        compute2(acc, f[kp & 1]);
      }
    } else {
#pragma unroll 1
      for (int kp = 0; kp < STEPS; ++kp) {
        Frag2 f;
        load_frag2(f, as, bs, KU * kp, ty, tx);
        compute2(acc, f);
      }
    }
  }

  static __device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int &bm, int &bn) {
    const int total = tiles_m * tiles_n;
    // consecutive workgroup ids land on consecutive XCDs (8 of them, one L2
    // each): give every XCD one contiguous run of the tile order
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr int GROUP = 8;
    const int width = GROUP * tiles_n;
    const int group = id / width, first = group * GROUP;
    const int gsz = min(tiles_m - first, GROUP);
    bm = first + (id % width) % gsz;
    bn = (id % width) / gsz;
  }

  // The workgroup's output tile and k range (blockIdx.y is the split-K slice).
  static __device__ __forceinline__ void tile_and_range(const Problem &p, int &m0, int &n0, int &kb, int &ke) {
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    int bm, bn;
    tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
    m0 = bm * BM;
    n0 = bn * BN;
    kb = 0;
    ke = p.k;
    if (p.workspace) {
      if (p.k_sub > 1) {
        // this workgroup's part of its slice: whole k-tiles, spread evenly over the slice's k_sub workgroups
        const int slice = blockIdx.y / p.k_sub, part = blockIdx.y % p.k_sub;
        const int sb = min(p.k, slice * p.k_per_slice), se = min(p.k, sb + p.k_per_slice);
        const int per = ((se - sb + BK - 1) / BK + p.k_sub - 1) / p.k_sub * BK;
        kb = min(se, sb + part * per);
        ke = min(se, kb + per);
      } else {
        kb = blockIdx.y * p.k_per_slice;
        ke = min(p.k, kb + p.k_per_slice);
      }
    }
  }
  // can the k range of a slice be shared out over several workgroups (Problem::k_sub)?  The parts meet in the
  // workspace through one native atomic per element, so: an add that has one, and accumulators that are final
  // as they stand (no mask to turn back, no zero whose sign depends on the rest of the range).
  static constexpr bool SUB_SLICES = has_native_fold<T, ADD>::value && !MASKED && !ZERO_SIGN;

  static __device__ __forceinline__ void run(const Problem &p, Smem &sm) {
    int m0, n0, kb, ke;
    tile_and_range(p, m0, n0, kb, ke);
    S acc[TM][TN];
    accumulate(p, sm, m0, n0, kb, ke, (ke - kb + BK - 1) / BK, acc);
    finish(p, acc, m0, n0, kb, ke);
  }

  // acc = identity, then the terms of k in [kb, ke).  The 256 threads that share `sm` pass
  // 1 + `sync_tiles` barriers (sync_tiles >= the number of k-tiles of the range, so that groups of
  // one workgroup whose ranges differ in length stay in step).
  static __device__ __forceinline__ void accumulate(const Problem &p, Smem &sm, int m0, int n0, int kb, int ke, int sync_tiles,
                                                    S (&acc)[TM][TN]) {
    const int tid = threadIdx.x & 255, tx = tid & 15, ty = tid >> 4;
    const T *A = reinterpret_cast<const T *>(p.A);
    const T *B = reinterpret_cast<const T *>(p.B);
    const T ident = scalar_as<T>(p.add_identity);
    const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;

#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = staged(ident);

    const int ntiles = max((ke - kb + BK - 1) / BK, 0);
    T ra[A_ELEMS], rb[B_ELEMS];
    Mover<BM, A_ELEMS> ma;
    Mover<BN, B_ELEMS> mb;
    if constexpr (VEC) {
      ma.init(A, p.sa_m, p.sa_k, m0, p.m, kb, a_xc);
      mb.init(B, p.sb_n, p.sb_k, n0, p.n, kb, b_xc);
    }
    // k-tile starting at k0 into registers
    auto fetch = [&](int k0) {
      if constexpr (VEC) {
        const int kcount = ke - k0;
        if (CAREFUL || kcount >= BK) {
          ma.load(ra);
          mb.load(rb);
        } else {
          ma.load_ragged(ra, p.sa_k, kcount, a_xc);
          mb.load_ragged(rb, p.sb_k, kcount, b_xc);
        }
      } else {
        load_panel<BM, A_ELEMS>(ra, A, p.sa_m, p.sa_k, m0, p.m, k0, ke, a_xc);
        load_panel<BN, B_ELEMS>(rb, B, p.sb_n, p.sb_k, n0, p.n, k0, ke, b_xc);
      }
    };
    // On the vector path the last k-tile of the workgroup is never fetched through the movers
    // (see Mover): fill_last puts it straight into its LDS stage -- which is free as soon as the
    // barrier that ended the previous iteration has been passed, so it is filled ahead of the
    // compute like a prefetch.
    auto fill_last_tile = [&](int k0, int stage) {
      fill_last<BM, LDA>(sm.a[stage], A, p.sa_m, p.sa_k, m0, p.m, k0, ke, a_xc);
      fill_last<BN, LDB>(sm.b[stage], B, p.sb_n, p.sb_k, n0, p.n, k0, ke, b_xc);
    };
    // ... unless nothing about the last tile can reach past the matrix: it is a whole tile and no
    // vector straddles an edge (x-contiguous extents are multiples of the vector width)
    const bool careful_last = VEC && CAREFUL && !((ke - kb) % BK == 0 && (!a_xc || p.m % VW == 0) && (!b_xc || p.n % VW == 0));
    if (ntiles > 0) {
      if (careful_last && ntiles == 1) {
        fill_last_tile(kb, 0);
      } else {
        fetch(kb);
        store_panel<BM, LDA, A_ELEMS>(ra, sm.a[0], a_xc);
        store_panel<BN, LDB, B_ELEMS>(rb, sm.b[0], b_xc);
      }
    }
    __syncthreads();
    int buf = 0;
    for (int t = 0; t < sync_tiles; ++t) {
      if (t < ntiles) {
        const int k0 = kb + t * BK;
        const bool more = t + 1 < ntiles;
        const bool next_is_last = careful_last && t + 2 == ntiles;
        if (next_is_last) fill_last_tile(k0 + BK, buf ^ 1);
        else if (more) fetch(k0 + BK);
        const int kcount = min(BK, ke - k0);
        if (kcount == BK) {
          whole_tile(acc, sm.a[buf], sm.b[buf], ty, tx);
        } else {
#pragma unroll 1
          for (int kk = 0; kk < kcount; ++kk) step(acc, sm.a[buf], sm.b[buf], kk, ty, tx);
        }
        if (more && !next_is_last) {
          store_panel<BM, LDA, A_ELEMS>(ra, sm.a[buf ^ 1], a_xc);
          store_panel<BN, LDB, B_ELEMS>(rb, sm.b[buf ^ 1], b_xc);
        }
      }
      __syncthreads();
      buf ^= 1;
    }
  }

  // ---- epilogue: D = add(mult(alpha, acc), mult(beta, C)), or raw partials; [kb, ke) is the
  // k range the accumulators cover (ZERO_SIGN looks into it)
  // (row_step, row_first: only the rows i = row_first, row_first + row_step, ... of the thread's outputs)
  static __device__ __forceinline__ void finish(const Problem &p, S (&acc)[TM][TN], int m0, int n0, int kb, int ke,
                                                int row_step = 1, int row_first = 0) {
    const int tid = threadIdx.x & 255, tx = tid & 15, ty = tid >> 4;
    const T *A = reinterpret_cast<const T *>(p.A);
    const T *B = reinterpret_cast<const T *>(p.B);
    const T ident = scalar_as<T>(p.add_identity);
    T *out;
    long long ld_out;
    const bool partial = p.workspace != nullptr;
    EpilogueScalars<T> e;
    if (partial) {
      out = reinterpret_cast<T *>(p.workspace) + (long long)(p.k_sub > 1 ? blockIdx.y / p.k_sub : blockIdx.y) * p.m * p.n;
      ld_out = p.n;
      e.alpha = e.beta = e.ident = ident;
      e.source_needed = false;
    } else {
      out = reinterpret_cast<T *>(p.D);
      ld_out = p.ldd;
      e = resolve_scalars<T>(p, MUL);
    }
    if constexpr (SUB_SLICES) {
      if (partial && p.k_sub > 1) {
        // one of several workgroups on this slice's tile: fold into the partial tile, which the host has filled
        // with the additive identity
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int row = m0 + ty * VW + (i / VW) * 16 * VW + (i % VW);
          if (row >= p.m || i % row_step != row_first) continue;
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int col = n0 + tx * VW + (j / VW) * 16 * VW + (j % VW);
            if (col < p.n) native_fold<ADD>(out + (long long)row * ld_out + col, acc[i][j]);
          }
        }
        return;
      }
    }
    const T *C = reinterpret_cast<const T *>(p.C);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = m0 + ty * VW + (i / VW) * 16 * VW + (i % VW);
      if (row >= p.m || i % row_step != row_first) continue;
#pragma unroll
      for (int g = 0; g < GN; ++g) {
        const int col = n0 + tx * VW + g * 16 * VW;
        if (col >= p.n) continue;
        T v[VW];
#pragma unroll
        for (int c = 0; c < VW; ++c) {
          if constexpr (MASKED) {
            v[c] = acc[i][g * VW + c] ? T(1) : T(0);
          } else {
            v[c] = acc[i][g * VW + c];
            if constexpr (ZERO_SIGN) {
              if (v[c] == T(0) && ke > kb)
                v[c] = last_zero_product(A + (long long)row * p.sa_m + (long long)kb * p.sa_k, p.sa_k,
                                         B + (long long)min(col + c, p.n - 1) * p.sb_n + (long long)kb * p.sb_k, p.sb_k,
                                         ke - kb, v[c]);
            }
          }
        }
        if (!partial) {
#pragma unroll
          for (int c = 0; c < VW; ++c) v[c] = Op<MUL>::apply(e.alpha, v[c]);
          if (e.source_needed) {
            T src[VW];
            if (VEC && (!CAREFUL || col + VW <= p.n)) {
              const gvec_t t = *reinterpret_cast<const gvec_t *>(C + (long long)row * p.ldc + col);
#pragma unroll
              for (int c = 0; c < VW; ++c) src[c] = t[c];
            } else {
#pragma unroll
              for (int c = 0; c < VW; ++c) src[c] = C[(long long)row * p.ldc + min(col + c, p.n - 1)];
            }
#pragma unroll
            for (int c = 0; c < VW; ++c) v[c] = fold_epilogue<ADD, MUL>(v[c], Op<MUL>::apply(e.beta, src[c]));
          }
        }
        if (VEC && (!CAREFUL || col + VW <= p.n)) {
          gvec_t t;
#pragma unroll
          for (int c = 0; c < VW; ++c) t[c] = v[c];
          *reinterpret_cast<gvec_t *>(out + (long long)row * ld_out + col) = t;
        } else {
#pragma unroll
          for (int c = 0; c < VW; ++c)
            if (col + c < p.n) out[(long long)row * ld_out + col + c] = v[c];
        }
      }
      __builtin_amdgcn_sched_barrier(0);  // one row of C in flight at a time
    }
  }
};

template <typename T, int ADD, int MUL, int TM, int TN, int BK, bool VEC, bool CAREFUL = false>
__global__ __launch_bounds__(256) WAVES_ATTR void valu_srgemm_kernel(Problem p) {
  using Tile = ValuTile<T, ADD, MUL, TM, TN, BK, VEC, CAREFUL>;
  __shared__ typename Tile::Smem sm;
  select_batch<T>(p);
  Tile::run(p, sm);
}

// The same tile with the k range shared out inside the workgroup, for launches that would
// otherwise leave most of the chip idle (an output of 1024^2 is 256 quarter-size tiles: one
// workgroup per compute unit, one wave per SIMD, and a single wave issues at little more than a
// third of the rate two or four reach).  G groups of 256 threads each take a run of whole k-tiles
// of the workgroup's range, with LDS panels of their own; the groups' accumulators then meet in LDS
// and group 0 folds them in ascending k order, acc = add(acc, partial) as the split-K reduction does,
// and runs the epilogue.  Only for adds whose result does not depend on how the terms are grouped
// (everything but a floating-point sum).
template <typename T, int ADD> struct order_free : std::integral_constant<bool, !(ADD == kPlus && is_fp<T>::value)> {};

template <typename T, int ADD, int MUL, int TM, int TN, int BK, bool VEC, bool CAREFUL, int G>
__global__ __launch_bounds__(256 * G) void valu_ksplit_kernel(Problem p) {
  using Tile = ValuTile<T, ADD, MUL, TM, TN, BK, VEC, CAREFUL>;
  using S = typename Tile::S;
  static_assert(order_free<T, ADD>::value, "a floating-point sum depends on the grouping of its terms");
  static_assert(G * sizeof(typename Tile::Smem) >= (G - 1) * sizeof(S) * TM * TN * 256 && TM % G == 0, "the groups' accumulators must fit the panel space");
  __shared__ typename Tile::Smem sm[G];
  select_batch<T>(p);
  const int g = threadIdx.x >> 8, tid = threadIdx.x & 255;
  int m0, n0, kb, ke;
  Tile::tile_and_range(p, m0, n0, kb, ke);
  const int tiles = max((ke - kb + BK - 1) / BK, 0), per = (tiles + G - 1) / G;
  const int gkb = min(ke, kb + g * per * BK), gke = min(ke, gkb + per * BK);
  S acc[TM][TN];
  Tile::accumulate(p, sm[g], m0, n0, gkb, gke, per, acc);  // ends with a barrier: every group is done with its panels
  // The panels are dead now.  Group d takes the rows i = d, d + G, ... of the threads' outputs: every group leaves
  // its accumulators of the other groups' rows in the panel space, and each group then folds its rows over the
  // groups in ascending k order (acc = add(acc, partial), as the split-K reduction does) and runs their epilogue --
  // one G-th of the fold, of the reads of C and of the stores each.
  // Where group h's row i (of group i % G != h) lies: rows in the order of i, without h's own
  constexpr int ROWS_OUT = TM - TM / G, AREA = ROWS_OUT * TN * 256;
  auto slot = [](int h, int i) { return (i / G) * (G - 1) + (i % G < h ? i % G : i % G - 1); };
  S *area = reinterpret_cast<S *>(&sm[0]);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (i % G == g) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) area[g * AREA + (slot(g, i) * TN + j) * 256 + tid] = acc[i][j];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (i % G != g) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      S v = acc[i][j];  // (overwritten unless g == 0)
#pragma unroll
      for (int h = 0; h < G; ++h) {
        if (h == i % G) {  // this row's own group: from its registers
          if (h > 0) {
            if constexpr (Tile::MASKED) v |= acc[i][j];
            else v = Op<ADD>::apply(v, acc[i][j]);
          }
        } else {
          const S w = area[h * AREA + (slot(h, i) * TN + j) * 256 + tid];
          if (h == 0) v = w;
          else if constexpr (Tile::MASKED) v |= w;
          else v = Op<ADD>::apply(v, w);
        }
      }
      acc[i][j] = v;
    }
  }
  Tile::finish(p, acc, m0, n0, kb, ke, G, g);
}

// Extents along every contiguous direction are multiples of the vector width: no vector straddles
// an edge, rows of D hold whole vectors (alignment itself is not needed: 16-byte accesses are legal
// at any element boundary).
template <typename T> static bool vector_exact(const Problem &p) {
  constexpr int VW = 16 / sizeof(T);
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;
  if (a_xc ? p.m % VW : (p.sa_k != 1 || p.k % VW)) return false;
  if (b_xc ? p.n % VW : (p.sb_k != 1 || p.k % VW)) return false;
  return p.n % VW == 0 && p.k >= 1;
}
// The careful vector path takes any extent; it only needs one whole vector inside each operand
// along its contiguous direction, for the vectors that lie wholly outside to point at.
template <typename T> static bool vector_possible(const Problem &p) {
  constexpr int VW = 16 / sizeof(T);
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;
  if (!a_xc && p.sa_k != 1) return false;  // neither direction contiguous (not produced by the C ABI)
  if (!b_xc && p.sb_k != 1) return false;
  if (a_xc && p.m < VW) return false;
  if (b_xc && p.n < VW) return false;
  return p.k >= 1;
}

// grid dimension y: one workgroup per slice, or k_sub per slice
static inline unsigned slice_groups(const Problem &p) { return p.workspace ? (unsigned)(p.slices * (p.k_sub > 1 ? p.k_sub : 1)) : 1u; }

template <typename T, int ADD, int MUL, int TM, int TN, int BK, int G>
static void launch_ksplit(const Problem &p, dim3 grid, hipStream_t s) {
  if (vector_exact<T>(p))
    launch_kernel((valu_ksplit_kernel<T, ADD, MUL, TM, TN, BK, true, false, G>), grid, dim3(256 * G), 0, s, p);
  else
    launch_kernel((valu_ksplit_kernel<T, ADD, MUL, TM, TN, BK, true, true, G>), grid, dim3(256 * G), 0, s, p);
}

#ifndef CUASR_AMD_KSPLIT2_MAX
#define CUASR_AMD_KSPLIT2_MAX 1024
#endif
// KSPLIT: this tile may share its k range out inside the workgroup when the launch is small.
template <typename T, int ADD, int MUL, int TM, int TN, int BK, bool KSPLIT = false>
static hipError_t launch_valu(const Problem &p, hipStream_t s) {
  constexpr int BM = 16 * TM, BN = 16 * TN;
  if (p.m == 0 || p.n == 0) return hipSuccess;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, slice_groups(p), p.batch);
  if constexpr (KSPLIT && order_free<T, ADD>::value) {
    // 256 compute units: up to 256 workgroups get four groups (1024 threads, four waves per SIMD),
    // up to 512 two; each group wants a few k-tiles of its own to be worth the fold at the end
    const long long groups = tiles * grid.y * grid.z;
    const long long k_range = p.workspace ? p.k_per_slice / (p.k_sub > 1 ? p.k_sub : 1) : p.k;
    if (vector_possible<T>(p) && k_range >= 8LL * BK) {
      if (groups <= 256) {
        launch_ksplit<T, ADD, MUL, TM, TN, BK, 4>(p, grid, s);
        return take_launch_status();
      }
      if (groups <= CUASR_AMD_KSPLIT2_MAX) {
        launch_ksplit<T, ADD, MUL, TM, TN, BK, 2>(p, grid, s);
        return take_launch_status();
      }
    }
  }
  if (vector_exact<T>(p))
    launch_kernel((valu_srgemm_kernel<T, ADD, MUL, TM, TN, BK, true, false>), grid, dim3(256), 0, s, p);
  else if (vector_possible<T>(p))
    launch_kernel((valu_srgemm_kernel<T, ADD, MUL, TM, TN, BK, true, true>), grid, dim3(256), 0, s, p);
  else
    launch_kernel((valu_srgemm_kernel<T, ADD, MUL, TM, TN, BK, false, false>), grid, dim3(256), 0, s, p);
  return take_launch_status();
}

// The chip holds 1024 full-size workgroups at a time (four per compute unit),
// and a launch runs in rounds of that many.  The full-size tile is a few per
// cent faster than the quarter-size one when its workgroups fill whole rounds
// (4096^2: exactly one), and much slower when a round is mostly empty (fewer
// than 1024 workgroups: split-K of a small output, matrices below ~3000^2) or
// the last round is (5120^2: 1.56 rounds).  The quarter-size tile -- four times
// as many, shorter workgroups -- balances in all those cases, so the full-size
// one is used only when at least 95 % of its rounds are filled.
#ifndef CUASR_AMD_FULL_TILE_FILL_PERCENT
#define CUASR_AMD_FULL_TILE_FILL_PERCENT 95
#endif

template <typename T, int ADD, int MUL, int TM, int TN, int BK, int TM_SMALL, int TN_SMALL, int BK_SMALL = BK>
static hipError_t launch_valu_sized(const Problem &p, hipStream_t s) {
  constexpr int BM = 16 * TM, BN = 16 * TN;
  const long long groups = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN) * slice_groups(p) * p.batch;
  const long long rounds = (groups + 1023) / 1024;
  if constexpr (order_free<T, ADD>::value) {
    // 192 .. 256 full-size workgroups (2048^2: exactly 256) are one per compute unit for most of the
    // chip: two groups per workgroup give every SIMD its two waves, and the full-size tile then runs
    // at the rate it has on large problems, which the quarter-size tile does not reach
    const long long k_range = p.workspace ? p.k_per_slice / (p.k_sub > 1 ? p.k_sub : 1) : p.k;
    if (groups >= 192 && groups <= 256 && k_range >= 8LL * BK && vector_possible<T>(p) && p.m > 0 && p.n > 0) {
      launch_ksplit<T, ADD, MUL, TM, TN, BK, 2>(p, dim3((unsigned)(groups / slice_groups(p) / p.batch), slice_groups(p), p.batch), s);
      return take_launch_status();
    }
  }
  if (groups * 100 < rounds * 1024 * (long long)(CUASR_AMD_FULL_TILE_FILL_PERCENT))
    return launch_valu<T, ADD, MUL, TM_SMALL, TN_SMALL, BK_SMALL, true>(p, s);
  return launch_valu<T, ADD, MUL, TM, TN, BK>(p, s);
}

}  // namespace cuasr_amd
