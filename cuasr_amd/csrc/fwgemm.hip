// Min-plus product that also records where each new minimum came from
// (the building block of all-pairs shortest paths with path recovery), and the
// repeated-squaring driver on top of it.  Semantics: cpu_fwgemm_naive,
// test/regress/include/fwgpu/cpu_srgemm.hpp:20-48 -- for every (row, col), scan
// k ascending, take prod = A[row,k] + B[k,col], and on prod < dist replace dist
// by prod and parent by k.  All four matrices are column-major.
//
// The result does not depend on the scan order when stated as: let v be the
// smallest product; if v < dist then dist = v and parent = the smallest k whose
// product equals v; otherwise nothing changes.  The tile kernel uses that form:
//   - per chunk of BK k-values it keeps a plain min-plus accumulator (1.5
//     vector instructions per term, as in the SRGEMM tiles),
//   - after the chunk, "chunk minimum < running minimum" (strict) moves the
//     running minimum and records the chunk index: 3 instructions per BK terms,
//   - the epilogue re-reads the recorded chunk of every improved element and
//     takes the first k whose product equals the minimum.  The product is the
//     same single addition of the same operands, so equality is exact, and the
//     stored distance is that product, which keeps the sign of a zero as the
//     sequential scan would.
// Operands must be free of NaN and of -infinity (+infinity marks "no edge").
#include "direct_tile.h"
#include "semiring.h"

#include <limits>
#include <type_traits>

namespace cuasr_amd {
namespace {

struct FwArgs {
  int m, n, k;
  const void *A; int64_t lda;
  const void *B; int64_t ldb;
  void *dist; int64_t ldc;
  int32_t *parent; int64_t ldp;
  // optional second image of A with k contiguous (At[row * ldat + k] = A[row, k]); the tile
  // kernel's lookup of the first minimising k then reads one run of memory per element
  // instead of one element from each of BK columns
  const void *At; int64_t ldat;
  int k_base;                               // recorded parents are k_base + k
  int skip_r0, skip_r1, skip_c0, skip_c1;   // outputs in these rows or these columns are left alone
  // one-thread-per-element and row-by-four-columns kernels only: every output they compute is also stored transposed,
  // out_t[col + row * ld_out_t] (the k-contiguous image a later product's lookups read)
  void *out_t; int64_t ld_out_t;
  // tile kernel, blocked Floyd-Warshall only: the diagonal block that starts at (ahead0, ahead0) and has
  // ahead_bb (> 0) rows is the next block step's and has had this step's update already: the launch's
  // first workgroup closes its distances (fw_close_dist) while the others do the product, which leaves that
  // block alone.  hist: 3 x FW_BLOCK x FW_BLOCK elements that take what fw_parents_block needs afterwards.
  int ahead0, ahead_bb;
  void *hist;
};

// cond ? a : b with a hidden from the optimiser: `x < y ? x : y` on floating point is
// folded into a hardware minimum when NaNs need not be honoured, and that minimum
// prefers -0 to +0, where the reference's comparison keeps whichever came first
template <typename T> __device__ __forceinline__ T pick(bool cond, T a, T b) {
  asm("" : "+v"(a));
  return cond ? a : b;
}

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N - 1>): a loop whose index is a compile-time constant
template <int N, int I = 0, typename F> __device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

// one thread per element, the literal scan; any extent, any leading dimension
template <typename T> __device__ __forceinline__ void fwgemm_naive_block(const FwArgs &g, int bx, int by) {
  const int row = bx * 64 + (threadIdx.x & 63);
  // (a wave's 64 threads share a column: saying so keeps B's addresses in scalar registers)
  const int col = __builtin_amdgcn_readfirstlane(by * 4 + (threadIdx.x >> 6));
  if (row >= g.m || col >= g.n) return;
  if ((row >= g.skip_r0 && row < g.skip_r1) || (col >= g.skip_c0 && col < g.skip_c1)) return;
  const T *a = static_cast<const T *>(g.A) + row;
  const T *b = static_cast<const T *>(g.B) + col * g.ldb;
  T *d = static_cast<T *>(g.dist) + row + col * g.ldc;
  int32_t *pp = g.parent + row + col * g.ldp;
  T curr = *d;
  int32_t p = *pp;
  int i = 0;
  for (; i + 16 <= g.k; i += 16) {  // sixteen k at a time, their operands requested together
    T av[16], bv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      av[u] = a[(i + u) * g.lda];
      bv[u] = b[i + u];
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const T prod = av[u] + bv[u];
      const bool lower = prod < curr;
      curr = pick(lower, prod, curr);
      p = lower ? g.k_base + i + u : p;
    }
  }
  for (; i < g.k; ++i) {
    const T prod = a[i * g.lda] + b[i];
    const bool lower = prod < curr;
    curr = pick(lower, prod, curr);
    p = lower ? g.k_base + i : p;
  }
  *d = curr;
  *pp = p;
  if (g.out_t) static_cast<T *>(g.out_t)[col + int64_t(row) * g.ld_out_t] = curr;
}

template <typename T>
__global__ void __launch_bounds__(256) fwgemm_naive_kernel(FwArgs g) {
  fwgemm_naive_block<T>(g, blockIdx.x, blockIdx.y);
}

template <typename T> struct vec4_of;
template <> struct vec4_of<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct vec4_of<double> { typedef double type __attribute__((ext_vector_type(4))); };

// One thread per output row and four columns, for products too small for the tile kernel but on the
// critical path (the block row and the block column of a blocked Floyd-Warshall step): a workgroup of 256
// threads covers 64 rows x 16 columns.  Same order-free form as the tile kernel: per chunk of 16 k a plain
// min-plus (a 3-input minimum per two products), and "chunk minimum < running minimum" (strict) moves the
// running minimum.  A chunk in which any of the wave's 64 rows improved is resolved on the spot, from the
// operands still in registers: the first k whose product equals the chunk minimum (the same single addition
// of the same operands, so equality is exact) is the parent, and that product, sign of zero included, the
// distance.  (Looking the chunk up after the loop, as the tile kernel does, costs a gather of 16 cache lines
// per lane and column here: 27 us for the two panels at n = 4096.)  A's 16 values of a chunk serve four
// columns.  The one-thread-per-element scan spends four instructions per term, two of which read a mask, and reads each A
// value once per output column: 29 us.
template <typename T> __device__ __forceinline__ void fwgemm_rowcols_block(const FwArgs &g, int bx, int by) {
  constexpr int CK = 16, NC = 4;
  const int row_of_lane = bx * 64 + (threadIdx.x & 63);
  const int col0 = __builtin_amdgcn_readfirstlane(by * 16 + (threadIdx.x >> 6) * NC);
  if (col0 >= g.n) return;  // (the whole wave)
  // every lane stays to the end, because every lane fetches one of the chunk's B values for the wave: rows
  // beyond the matrix or in the skipped range are computed on a clamped row and never stored
  const bool row_live = row_of_lane < g.m && !(row_of_lane >= g.skip_r0 && row_of_lane < g.skip_r1);
  const int row = row_of_lane < g.m ? row_of_lane : g.m - 1;
  const T inf = std::numeric_limits<T>::infinity();
  const int64_t lda = g.lda;
  // columns beyond the matrix or in the skipped range: computed on a clamped column, never stored
  int64_t out[NC];
  bool live[NC];
  T curr[NC];
  int32_t par[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int cc = col0 + c, cl = cc < g.n ? cc : g.n - 1;
    live[c] = row_live && cc < g.n && !(cc >= g.skip_c0 && cc < g.skip_c1);
    out[c] = cl;
    curr[c] = static_cast<const T *>(g.dist)[row + int64_t(cl) * g.ldc];
    par[c] = -1;
  }
  // one chunk of CK k-values; FULL: all of them exist (the ragged last chunk takes +infinity for the others,
  // which neither improves anything nor equals a minimum that did)
  // B's 4 x 16 values of a chunk: one load per lane (lane = column, k), handed round through a piece of LDS that
  // belongs to the wave (no barrier: a wave's LDS accesses complete in order) and read back as broadcasts.
  // Through scalar loads instead, every chunk and column waited for a scalar-cache miss, and every add read
  // a scalar register, which costs it a second issue slot.
  __shared__ T bstage[4][2][NC * CK];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T *blane = static_cast<const T *>(g.B) + int64_t(min(col0 + (lane >> 4), g.n - 1)) * g.ldb;
  const T *ap = static_cast<const T *>(g.A) + row;
  auto load = [&](T (&av)[CK], T &bl, int k0, auto full) {
    constexpr bool FULL = decltype(full)::value;
    bl = blane[FULL ? k0 + (lane & 15) : min(k0 + (lane & 15), g.k - 1)];
#pragma unroll
    for (int u = 0; u < CK; ++u) {
      if constexpr (FULL) av[u] = *ap;
      else av[u] = k0 + u < g.k ? *ap : inf;
      if (FULL || k0 + u + 1 < g.k) ap += lda;
    }
  };
  auto compute = [&](const T (&av)[CK], T bl, int k0, int buf) {
    typedef typename vec4_of<T>::type V4;
    bstage[wave][buf][lane] = bl;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      T bv[CK];
#pragma unroll
      for (int q = 0; q < CK / 4; ++q) {
        const V4 v = *reinterpret_cast<const V4 *>(&bstage[wave][buf][c * CK + q * 4]);
#pragma unroll
        for (int e = 0; e < 4; ++e) bv[q * 4 + e] = v[e];
      }
      T prod[CK], best = inf;
#pragma unroll
      for (int u = 0; u < CK; ++u) prod[u] = av[u] + bv[u];
#pragma unroll
      for (int u = 0; u < CK; u += 2) best = hw_min<T>(hw_min<T>(best, prod[u]), prod[u + 1]);
      const bool lower = best < curr[c];
      if (__builtin_amdgcn_ballot_w64(lower)) {  // the same for the whole wave
        int first = 0;
#pragma unroll
        for (int u = CK - 1; u >= 0; --u) first = prod[u] == best ? u : first;
        T value = best;
        // a minimum of zero: the hardware's may carry the other sign than the first product that equals it
        if (__builtin_amdgcn_ballot_w64(lower && best == T(0))) {
#pragma unroll
          for (int u = CK - 1; u >= 0; --u) value = pick(prod[u] == best, prod[u], value);
        }
        curr[c] = lower ? value : curr[c];
        par[c] = lower ? g.k_base + k0 + first : par[c];
      }
    }
  };
  // the next chunk's A values are requested before this chunk is worked on: a wave has eight chunks and a
  // compute unit sixteen such waves, too few to hide a memory round trip per chunk behind each other
  const int nfull = g.k / CK;
  T av[2][CK], bl[2];
  if (nfull > 0) load(av[0], bl[0], 0, std::true_type{});
  for (int ch = 0; ch < nfull; ch += 2) {
    if (ch + 1 < nfull) load(av[1], bl[1], (ch + 1) * CK, std::true_type{});
    compute(av[0], bl[0], ch * CK, 0);
    if (ch + 1 < nfull) {
      if (ch + 2 < nfull) load(av[0], bl[0], (ch + 2) * CK, std::true_type{});
      compute(av[1], bl[1], (ch + 1) * CK, 1);
    }
  }
  if (nfull * CK < g.k) {
    load(av[0], bl[0], nfull * CK, std::false_type{});
    compute(av[0], bl[0], nfull * CK, 0);
  }
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    if (!live[c]) continue;
    if (par[c] >= 0) {
      static_cast<T *>(g.dist)[row + out[c] * g.ldc] = curr[c];
      g.parent[row + out[c] * g.ldp] = par[c];
    }
    if (g.out_t) static_cast<T *>(g.out_t)[out[c] + int64_t(row) * g.ld_out_t] = curr[c];
  }
}

// The improved elements of a tile, queued in LDS as (code = row in the tile | column << ROW_BITS | chunk <<
// (ROW_BITS + COL_BITS), minimum), are looked up by groups of CHUNK / 4 lanes: each lane adds four of the chunk's
// products (one 16- or 32-byte load from B's column and one from the k-contiguous image of A), the group agrees on
// the first k whose product equals the minimum, and the lane that holds it stores that product -- the same single
// addition of the same operands as in the main loop, so the comparison is exact and the stored distance has the sign
// that the sequential scan would leave -- and the predecessor.  A wave's load then touches one cache line per
// element where one lane per element would touch 64.  A group takes UN elements per turn and requests all their
// operands before it looks at any: a turn costs one round trip to memory, and a tile has few turns.
template <int G> __device__ __forceinline__ int group_min(int v) {
  // minimum over the G (4 or 8) adjacent lanes of a group, by data-parallel moves inside the row of 16 lanes
  v = min(v, __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, true));   // lanes 1 0 3 2 of each four
  v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, true));   // lanes 2 3 0 1 of each four
  if constexpr (G == 8) v = min(v, __builtin_amdgcn_update_dpp(v, v, 0x141, 0xf, 0xf, true));  // each eight mirrored
  return v;
}
template <typename T, int THREADS, int CHUNK, bool HAS_AT, int ROW_BITS, int COL_BITS>
__device__ __forceinline__ void lookup_queue(const FwArgs &g, const uint32_t *q_code, const T *q_want, int count, int tid,
                                             int m0, int n0) {
  typedef typename vec4_of<T>::type V4;
  constexpr int G = CHUNK / 4, GROUPS = THREADS / G;
  constexpr int UN = sizeof(T) == 4 ? 8 : 4;
  static_assert(G == 4 || G == 8, "lanes per element");
  const T *A = static_cast<const T *>(g.A), *B = static_cast<const T *>(g.B), *At = static_cast<const T *>(g.At);
  T *dist = static_cast<T *>(g.dist);
  const int sub = tid % G;
  for (int e0 = tid / G; e0 < count; e0 += UN * GROUPS) {
    int r[UN], c[UN], k0[UN];
    T want[UN];
    V4 pa[UN], pb[UN];
    bool live[UN];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int e = e0 + u * GROUPS;
      live[u] = e < count;
      const uint32_t code = q_code[live[u] ? e : e0];  // (a turn's last elements may not exist: their lanes look at the first again)
      want[u] = q_want[live[u] ? e : e0];
      r[u] = m0 + int(code & ((1u << ROW_BITS) - 1));
      c[u] = n0 + int((code >> ROW_BITS) & ((1u << COL_BITS) - 1));
      k0[u] = int(code >> (ROW_BITS + COL_BITS)) * CHUNK + 4 * sub;
      pb[u] = *reinterpret_cast<const V4 *>(B + k0[u] + int64_t(c[u]) * g.ldb);
      if constexpr (HAS_AT) {
        pa[u] = *reinterpret_cast<const V4 *>(At + k0[u] + int64_t(r[u]) * g.ldat);
      } else {
#pragma unroll
        for (int x = 0; x < 4; ++x) pa[u][x] = A[r[u] + int64_t(k0[u] + x) * g.lda];
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      T value = want[u];
      int first = 4;
#pragma unroll
      for (int x = 3; x >= 0; --x) {
        const T prod = pa[u][x] + pb[u][x];
        const bool hit = prod == want[u];
        first = hit ? x : first;
        value = pick(hit, prod, value);
      }
      const int key = first < 4 ? 4 * sub + first : CHUNK;  // where in the chunk my first hit is
      const int best = group_min<G>(key);
      if (live[u] && first < 4 && key == best) {
        dist[r[u] + int64_t(c[u]) * g.ldc] = value;
        g.parent[r[u] + int64_t(c[u]) * g.ldp] = g.k_base + k0[u] + first;
      }
    }
  }
}

// 256 threads as 16 x 16; each owns TM x TN outputs in groups of four rows /
// columns that lie 64 apart, so a workgroup covers (16 TM) x (16 TN).
// GUARD = false: whole tiles, 16-byte aligned columns of A and B (vector loads).
// GUARD = true : any extents and alignment; out-of-range operands read as
//                +infinity, whose products never improve anything.
template <typename T, int TM, int TN, int SN, int BK, bool GUARD, bool HAS_AT>
__device__ __forceinline__ void fwgemm_tile_body(const FwArgs &g, const int block_x, const int block_y) {
  typedef typename vec4_of<T>::type V4;
  constexpr int BM = 16 * TM, BN = 16 * TN, PAD = 4;
  constexpr int NA = BM * BK / 4 / 256, NB = BN * BK / 4 / 256;
  static_assert(TM % 4 == 0 && TN % SN == 0 && SN % 4 == 0 && BK % 4 == 0 && BK % 2 == 0 && NA >= 1 && NB >= 1, "tile shape");
  __shared__ __attribute__((aligned(16))) T as[2][BK][BM + PAD];
  __shared__ __attribute__((aligned(16))) T bs[2][BK][BN + PAD];

  const T *A = static_cast<const T *>(g.A);
  const T *B = static_cast<const T *>(g.B);
  const int tid = threadIdx.x & 255;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = block_x * BM, n0 = block_y * BN;
  // (the host only passes ranges whose ends fall on tile boundaries or beyond the matrix)
  if ((m0 < g.skip_r1 && m0 + BM > g.skip_r0) || (n0 < g.skip_c1 && n0 + BN > g.skip_c0)) return;
  const T inf = std::numeric_limits<T>::infinity();

  auto row_of = [&](int i) { return m0 + (i >> 2) * 64 + tx * 4 + (i & 3); };
  auto col_of = [&](int j) { return n0 + (j >> 2) * 64 + ty * 4 + (j & 3); };

  V4 ra[NA], rb[NB];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int p = 0; p < NA; ++p) {
      const int v = tid + p * 256, r = (v % (BM / 4)) * 4, kk = v / (BM / 4);
      if constexpr (!GUARD) {
        ra[p] = *reinterpret_cast<const V4 *>(A + (m0 + r) + int64_t(k0 + kk) * g.lda);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          ra[p][e] = (m0 + r + e < g.m && k0 + kk < g.k) ? A[(m0 + r + e) + int64_t(k0 + kk) * g.lda] : inf;
      }
    }
#pragma unroll
    for (int p = 0; p < NB; ++p) {
      const int v = tid + p * 256, kk = (v % (BK / 4)) * 4, c = v / (BK / 4);
      if constexpr (!GUARD) {
        rb[p] = *reinterpret_cast<const V4 *>(B + (k0 + kk) + int64_t(n0 + c) * g.ldb);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          rb[p][e] = (n0 + c < g.n && k0 + kk + e < g.k) ? B[(k0 + kk + e) + int64_t(n0 + c) * g.ldb] : inf;
      }
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int p = 0; p < NA; ++p) {
      const int v = tid + p * 256, r = (v % (BM / 4)) * 4, kk = v / (BM / 4);
      *reinterpret_cast<V4 *>(&as[buf][kk][r]) = ra[p];
    }
#pragma unroll
    for (int p = 0; p < NB; ++p) {
      const int v = tid + p * 256, kk = (v % (BK / 4)) * 4, c = v / (BK / 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) bs[buf][kk + e][c] = rb[p][e];
    }
  };

  struct Frag {
    T a[2][4], b[2][SN];
  };
  auto load_frag = [&](Frag &f, int buf, int kk, int qi, int qj) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      *reinterpret_cast<V4 *>(&f.a[u][0]) = *reinterpret_cast<const V4 *>(&as[buf][kk + u][qi * 64 + tx * 4]);
#pragma unroll
      for (int q = 0; q < SN / 4; ++q)
        *reinterpret_cast<V4 *>(&f.b[u][q * 4]) =
            *reinterpret_cast<const V4 *>(&bs[buf][kk + u][(qj * (SN / 4) + q) * 64 + ty * 4]);
    }
  };

  T acc[TM][TN];
  int32_t chunk[TM][TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int r = row_of(i), c = col_of(j);
      chunk[i][j] = -1;
      if constexpr (!GUARD) acc[i][j] = static_cast<const T *>(g.dist)[r + int64_t(c) * g.ldc];
      else acc[i][j] = (r < g.m && c < g.n) ? static_cast<const T *>(g.dist)[r + int64_t(c) * g.ldc] : -inf;
    }
  if constexpr (!GUARD) {
    // a lane's rows come in runs of four: one 16-byte load per run when dist allows it
    const size_t vb = 4 * sizeof(T);
    if (reinterpret_cast<uintptr_t>(g.dist) % vb == 0 && g.ldc % 4 == 0) {
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; i += 4) {
          const V4 v = *reinterpret_cast<const V4 *>(static_cast<const T *>(g.dist) + row_of(i) + int64_t(col_of(j)) * g.ldc);
#pragma unroll
          for (int x = 0; x < 4; ++x) acc[i + x][j] = v[x];
        }
    }
  }

  const int tiles = (g.k + BK - 1) / BK;
  if (tiles > 0) {
    fetch(0);
    stage(0);
  }
  __syncthreads();
  for (int t = 0; t < tiles; ++t) {
    const int cur = t & 1;
    if (t + 1 < tiles) fetch((t + 1) * BK);
    // one block of 4 x SN outputs at a time, so that only its chunk minima are live
#pragma unroll
    for (int qi = 0; qi < TM / 4; ++qi)
#pragma unroll
      for (int qj = 0; qj < TN / SN; ++qj) {
        T best[4][SN];
        // two k-values per step (a 3-input minimum per pair of products); the next
        // step's fragments are read from LDS while this one is computed, and the
        // scheduling barriers keep the reads of later steps from being hoisted
        // (a whole tile's fragments do not fit in registers)
        Frag f[2];
        load_frag(f[0], cur, 0, qi, qj);
#pragma unroll
        for (int kp = 0; kp < BK / 2; ++kp) {
          if (kp + 1 < BK / 2) load_frag(f[(kp + 1) & 1], cur, 2 * (kp + 1), qi, qj);
          __builtin_amdgcn_sched_barrier(0);
          const Frag &x = f[kp & 1];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < SN; ++j) {
              const T p0 = x.a[0][i] + x.b[0][j], p1 = x.a[1][i] + x.b[1][j];
              best[i][j] = kp == 0 ? hw_min<T>(p0, p1) : hw_min<T>(hw_min<T>(best[i][j], p0), p1);
              // ties the arithmetic to this place in the instruction order: without it
              // instruction selection emits it next to its only use, after every read
              asm volatile("" : "+v"(best[i][j]));
            }
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < SN; ++j) {
            T &running = acc[qi * 4 + i][qj * SN + j];
            int32_t &where = chunk[qi * 4 + i][qj * SN + j];
            const bool lower = best[i][j] < running;
            running = lower ? best[i][j] : running;
            where = lower ? t : where;
          }
      }
    if (t + 1 < tiles) stage(cur ^ 1);
    __syncthreads();
  }

  // improved elements: the first k of the recorded chunk whose product is the minimum
  T *dist = static_cast<T *>(g.dist);
  // the element addresses are formed again from a thread index the compiler cannot
  // match with the prologue's: keeping 2 x TM x TN addresses live across the loop
  // would push the accumulators out of the register file
  int tx2 = tx, ty2 = ty;
  asm volatile("" : "+v"(tx2), "+v"(ty2));
  if constexpr (!GUARD) {
    // Whole, aligned tiles.  Improved elements are few in most launches and scattered over the
    // lanes, so they are first collected in a queue in LDS (the panels are no longer needed) and the
    // queue is then worked off by all 256 threads (lookup_queue): no lane waits for an element that did
    // not improve.  The queue takes as many whole columns j of the lanes' outputs as fit (one column
    // always does: at most 256 x TM elements), so a tile with few improved elements -- the usual case --
    // is done in one round of queueing, barrier and lookups, not one per column.
    constexpr int CAP = (sizeof(as) / sizeof(int) < sizeof(bs) / sizeof(T) ? sizeof(as) / sizeof(int) : sizeof(bs) / sizeof(T)) / 256 * 256;
    static_assert(CAP >= 256 * TM && BM <= 128 && BN <= 128, "a column of the lanes' outputs must fit in the panels");
    // Where an element goes in the queue follows from counts alone, without a shared counter (whose every use is a
    // round trip to LDS that the next one waits for): column by column, inside a column wave by wave, inside a wave
    // row i by row i, inside a row lane by lane.  Each wave counts its improved elements per column first.
    __shared__ int wave_count[4][TN];
    uint32_t *q_code = reinterpret_cast<uint32_t *>(&as[0][0][0]);  // row | column << 7 | chunk << 14 (the host sees to k < 2^22)
    T *q_want = reinterpret_cast<T *>(&bs[0][0][0]);                // the minimum found
    const int wave = tid >> 6;
    __syncthreads();  // everybody is done with the panels
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int n_improved = 0;  // in this column, over the wave
#pragma unroll
      for (int i = 0; i < TM; ++i) n_improved += __builtin_popcountll(__builtin_amdgcn_ballot_w64(chunk[i][j] >= 0));
      if ((tid & 63) == 0) wave_count[wave][j] = n_improved;
    }
    __syncthreads();
    int before_me[TN], col_count[TN];  // improved elements of the column in the waves before mine / in all waves
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      before_me[j] = col_count[j] = 0;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int n = __builtin_amdgcn_readfirstlane(wave_count[w][j]);
        before_me[j] += w < wave ? n : 0;
        col_count[j] += n;
      }
    }
    for (int j0 = 0; j0 < TN;) {  // (the same for every thread)
      int total = 0, j1 = j0;
#pragma unroll
      for (int j = 0; j < TN; ++j) {  // as many whole columns from j0 on as fit
        if (j < j0 || j != j1) continue;
        if (j > j0 && total + col_count[j] > CAP) continue;
        total += col_count[j];
        j1 = j + 1;
      }
      if (total > 0) {
        int base = 0;  // of the column in the queue
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if (j < j0 || j >= j1) continue;
          int slot0 = base + before_me[j];  // of my wave's next row of this column
#pragma unroll
          for (int i = 0; i < TM; ++i) {
            const unsigned long long improved = __builtin_amdgcn_ballot_w64(chunk[i][j] >= 0);
            if (chunk[i][j] >= 0) {
              const int slot = slot0 + __builtin_amdgcn_mbcnt_hi(uint32_t(improved >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(improved), 0u));
              q_code[slot] = uint32_t((i >> 2) * 64 + tx2 * 4 + (i & 3)) | uint32_t((j >> 2) * 64 + ty2 * 4 + (j & 3)) << 7 |
                             uint32_t(chunk[i][j]) << 14;
              q_want[slot] = acc[i][j];
            }
            slot0 += __builtin_popcountll(improved);
          }
          base += col_count[j];
        }
        __syncthreads();
        lookup_queue<T, 256, BK, HAS_AT, 7, 7>(g, q_code, q_want, total, tid, m0, n0);
        __syncthreads();  // the queue is free again
      }
      j0 = j1;
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int c = n0 + (j >> 2) * 64 + ty2 * 4 + (j & 3);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int r = m0 + (i >> 2) * 64 + tx2 * 4 + (i & 3);
      const int ch = chunk[i][j];
      if (ch < 0) continue;
      if constexpr (GUARD) {
        if (r >= g.m || c >= g.n) continue;
      }
      const int k0 = ch * BK;
      const T *ap = HAS_AT ? static_cast<const T *>(g.At) + k0 + int64_t(r) * g.ldat : A + r + int64_t(k0) * g.lda;
      const int64_t a_step = HAS_AT ? 1 : g.lda;
      const T *bp = B + k0 + int64_t(c) * g.ldb;
      const T want = acc[i][j];
      T value = want;
      int first = 0;
#pragma unroll 4
      for (int kk = BK - 1; kk >= 0; --kk) {
        bool in = true;
        if constexpr (GUARD) in = k0 + kk < g.k;
        const T prod = in ? ap[int64_t(kk) * a_step] + bp[kk] : inf;
        const bool hit = in && prod == want;
        first = hit ? kk : first;
        value = pick(hit, prod, value);
      }
      dist[r + int64_t(c) * g.ldc] = value;
      g.parent[r + int64_t(c) * g.ldp] = g.k_base + k0 + first;
    }
  }
}

constexpr int FW_BLOCK = 128;  // vertices per block step of the blocked Floyd-Warshall

// ---- closing a diagonal block in two parts: distances first, predecessors afterwards
//
// Step k of the closure lowers d[i][j] to cand_k = d[i][k] + d[k][j] (row k and column k as they are before the
// step) wherever that is strictly smaller, and the predecessor of (i, j) is the last k that did so.  A step that
// lowers an element is a strict record of the sequence d0[i][j], cand_0, cand_1, ...; the last record of a
// sequence is the first place its minimum is at.  So, given the rows and columns that the steps read, the
// predecessors are those of one min-plus product with predecessor tracking (fwgemm's own semantics, strict
// comparison, k ascending) of a matrix whose column k is "column k before step k" with one whose row k is
// "row k before step k", started from the block as it was before the closure.  Nothing of that product is on the
// critical path: nothing that follows reads a diagonal block's predecessors, and the product is spread over 64
// workgroups of a later launch.
//
// What stays on the critical path is fw_close_dist: the 128 dependent steps for the distances alone, an addition
// and a minimum per element and step (half the instructions of a step that also selects predecessors, and none
// that reads a comparison mask), by one workgroup of 256 threads with an 8 x 8 patch per thread.  Every row and
// column that a step publishes to LDS for the next one also goes to hist (row k and column k as step k reads them),
// and the block as it was found goes there too.
//
// The hardware minimum prefers -0 to +0 where the strict comparison keeps whichever came first.  Sums and minima
// of data free of -0 never produce one, so the block is searched for a -0 when it is loaded, and a block with
// one is closed by fw_close_dist_exact instead: the same steps with a comparison and a select, the block in place.
//
// hist: FW_BLOCK x FW_BLOCK elements each of  col[k * FW_BLOCK + i] = d[i][k] before step k,
// row[k * FW_BLOCK + j] = d[k][j] before step k,  init[(8 * (i % 8) + j % 8) * 256 + i / 8 + 16 * (j / 8)] = d[i][j] before
// the closure.
// (returns false, with nothing done, when the block holds a -0)
// (A function of its own, not inlined: as part of a kernel that also holds the other form and a product's tile, the
// compiler's register allocation moves parts of the patch to scratch memory inside the step loop, where any wait for
// memory also waits for the stores to hist.  Alone, either form fits the registers.)
template <typename T>
__device__ __attribute__((noinline)) bool fw_close_dist_fast(T *d_anywhere, int64_t ld, int bb, T *hist_anywhere,
                                                           __attribute__((address_space(3))) T *colbuf,
                                                           __attribute__((address_space(3))) T *rowbuf) {
  typedef typename vec4_of<T>::type V4;
  typedef __attribute__((address_space(3))) T LT;
  typedef __attribute__((address_space(3))) V4 LV4;
  // (both are device memory, which a function that is not a kernel has to be told: a store to "memory of some
  // kind" counts as an LDS access as well, and the waits for LDS before each barrier would wait for it)
  typedef __attribute__((address_space(1))) T GT;
  typedef __attribute__((address_space(1))) V4 GV4;
  GT *const d = (GT *)d_anywhere, *const hist = (GT *)hist_anywhere;
  // colbuf, rowbuf: lines of FW_BLOCK elements in LDS for columns k (and k + 1) as the steps read them, and for
  // the rows: two sets of one line for 8-byte elements (lines 0 and 2), four sets of two lines for 4-byte elements
  const int tid = threadIdx.x & 255, ti = tid & 15, tj = tid >> 4;  // rows 8 ti .. 8 ti + 7, columns 8 tj .. 8 tj + 7
  const T inf = std::numeric_limits<T>::infinity();
  GT *hist_col = hist, *hist_row = hist + FW_BLOCK * FW_BLOCK, *init = hist + 2 * FW_BLOCK * FW_BLOCK;
  T cur[8][8];  // [row in patch][column in patch]
  // loads from clamped addresses, then a select (a branch per element would keep 64 lane masks alive); a column's
  // addresses differ by the clamped row, so that the 64 loads in flight do not need 64 addresses in registers
  int ic[8];
#pragma unroll
  for (int a = 0; a < 8; ++a) ic[a] = min(8 * ti + a, bb - 1);
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const int j = 8 * tj + b;
    const GT *column = d + int64_t(min(j, bb - 1)) * ld;
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      const T v = column[ic[a]];
      cur[a][b] = (8 * ti + a < bb && j < bb) ? v : inf;
    }
  }
  {
    // a block with a -0 is left to the other form (a function of its own too: as part of this one the registers
    // it needs would be taken from this one's loop)
    bool negative_zero = false;
#pragma unroll
    for (int b = 0; b < 8; ++b)
#pragma unroll
      for (int a = 0; a < 8; ++a) negative_zero |= cur[a][b] == T(0) && __builtin_signbit(cur[a][b]);
    if (__syncthreads_or(negative_zero)) return false;
  }
  // (element by element, a thread's elements 256 apart: written four at a time, the patch's registers would have
  // to be adjacent in fours, and the compiler moves parts of the patch to scratch memory over that in the loop below)
#pragma unroll
  for (int b = 0; b < 8; ++b)
#pragma unroll
    for (int a = 0; a < 8; ++a) init[(8 * a + b) * 256 + tid] = cur[a][b];
  // (the minimum as an instruction: from the builtin the compiler first "quiets" an operand whose origin it
  // does not know, such as anything that comes round the loop, an instruction more per element)
  auto relax = [](T &x, const T cand) {
    if constexpr (sizeof(T) == 4) asm("v_min_f32 %0, %0, %1" : "+v"(x) : "v"(cand));
    else asm("v_min_f64 %0, %0, %1" : "+v"(x) : "v"(cand));
  };
  // two steps' candidates at once, in the steps' order
  auto relax2 = [&](T &x, const T first, const T second) {
    if constexpr (sizeof(T) == 4) {
      asm("v_min3_f32 %0, %0, %1, %2" : "+v"(x) : "v"(first), "v"(second));
    } else {
      relax(x, first);
      relax(x, second);
    }
  };
  // Rows and columns go to LDS two elements per instruction, each from a register of its own: as 16-byte stores the
  // compiler wants every row of the patch AND every column of it in four adjacent registers, cannot have both, and
  // moves parts of the patch to scratch memory in the attempt.  colbuf / rowbuf: [2 * buffer + which of the pair]
  auto lds = [](const LT *q) { return (unsigned)(size_t)q; };
  auto write2 = [](unsigned addr, const T x, const T y, auto at) {
    constexpr int AT = decltype(at)::value;  // in elements
    if constexpr (sizeof(T) == 4) asm volatile("ds_write2_b32 %0, %1, %2 offset0:%3 offset1:%4" ::"v"(addr), "v"(x), "v"(y), "n"(AT), "n"(AT + 1) : "memory");
    else asm volatile("ds_write2_b64 %0, %1, %2 offset0:%3 offset1:%4" ::"v"(addr), "v"(x), "v"(y), "n"(AT), "n"(AT + 1) : "memory");
  };
  // row S of the patch to row_at, column S to col_at (S is a compile-time constant, the step loop being unrolled
  // by eight: indexed by a run-time value the patch would live in scratch memory)
  auto put_row = [&](unsigned row_at, auto sc, auto at) {
    constexpr int S = decltype(sc)::value, AT = decltype(at)::value;
    write2(row_at, cur[S][0], cur[S][1], std::integral_constant<int, AT + 0>{});
    write2(row_at, cur[S][2], cur[S][3], std::integral_constant<int, AT + 2>{});
    write2(row_at, cur[S][4], cur[S][5], std::integral_constant<int, AT + 4>{});
    write2(row_at, cur[S][6], cur[S][7], std::integral_constant<int, AT + 6>{});
  };
  auto put_col = [&](unsigned col_at, auto sc, auto at) {
    constexpr int S = decltype(sc)::value, AT = decltype(at)::value;
    write2(col_at, cur[0][S], cur[1][S], std::integral_constant<int, AT + 0>{});
    write2(col_at, cur[2][S], cur[3][S], std::integral_constant<int, AT + 2>{});
    write2(col_at, cur[4][S], cur[5][S], std::integral_constant<int, AT + 4>{});
    write2(col_at, cur[6][S], cur[7][S], std::integral_constant<int, AT + 6>{});
  };
  auto get8 = [&](T (&x)[8], const LT *from) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const V4 v = *reinterpret_cast<const LV4 *>(from + 4 * h);
#pragma unroll
      for (int e = 0; e < 4; ++e) x[4 * h + e] = v[e];
    }
  };
  auto put8 = [&](GT *to, const T (&x)[8]) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      V4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = x[4 * h + e];
      *reinterpret_cast<GV4 *>(to + 4 * h) = v;
    }
  };

  if constexpr (sizeof(T) == 8) {
    // ---- 8-byte elements: one step per barrier, in one part.  The patch takes half the register file, and a
    // second set of rows and columns on its way beside the one in use pushes parts of the patch into scratch
    // memory.  (The product beside this closure takes twice as long anyway.)
    const unsigned row_lds[2] = {lds(rowbuf + (0) * FW_BLOCK + 8 * tj), lds(rowbuf + (2) * FW_BLOCK + 8 * tj)};
    const unsigned col_lds[2] = {lds(colbuf + (0) * FW_BLOCK + 8 * ti), lds(colbuf + (2) * FW_BLOCK + 8 * ti)};
    T ci[8], rj[8];  // column k at my rows, row k at my columns, for the step in hand
    auto publish = [&](int kn, auto bufc, auto sc) {
      constexpr int BUF = decltype(bufc)::value;
      if ((kn >> 3) == ti) put_row(row_lds[BUF], sc, std::integral_constant<int, 0>{});  // my patch holds row kn
      if ((kn >> 3) == tj) put_col(col_lds[BUF], sc, std::integral_constant<int, 0>{});  // my patch holds column kn
      // (the barrier that follows is the compiler's, which does not know of the instructions above)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    // what step kn reads goes to hist from the registers of the threads of the first patch row / column, which
    // together have read all of it
    auto fetch = [&](int buf, int kn) {
      get8(ci, colbuf + (2 * buf) * FW_BLOCK + 8 * ti);
      get8(rj, rowbuf + (2 * buf) * FW_BLOCK + 8 * tj);
      if (kn >= FW_BLOCK) return;
      if (tj == 0) put8(&hist_col[kn * FW_BLOCK + 8 * ti], ci);
      if (ti == 0) put8(&hist_row[kn * FW_BLOCK + 8 * tj], rj);
    };
    auto step = [&](int k, auto uc) {
      constexpr int U = decltype(uc)::value;  // k & 7
#pragma unroll
      for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) relax(cur[a][b], ci[a] + rj[b]);
      __builtin_amdgcn_sched_barrier(0);
      // into the other pair of buffers: nobody reads it before the barrier, and nobody is still reading it
      // from the step before (everybody has passed that step's barrier, and used what it read before that)
      publish(k + 1, std::integral_constant<int, (U & 1) ^ 1>{}, std::integral_constant<int, (U + 1) & 7>{});
      __syncthreads();
      fetch((U & 1) ^ 1, k + 1);
      __builtin_amdgcn_sched_barrier(0);
    };
    publish(0, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
    __syncthreads();
    fetch(0, 0);
    // steps beyond bb (up to the next multiple of eight) read rows and columns of the padding, which hold
    // +infinity and improve nothing
#pragma unroll 1
    for (int k8 = 0; k8 < bb; k8 += 8) {
      step(k8 + 0, std::integral_constant<int, 0>{});
      step(k8 + 1, std::integral_constant<int, 1>{});
      step(k8 + 2, std::integral_constant<int, 2>{});
      step(k8 + 3, std::integral_constant<int, 3>{});
      step(k8 + 4, std::integral_constant<int, 4>{});
      step(k8 + 5, std::integral_constant<int, 5>{});
      step(k8 + 6, std::integral_constant<int, 6>{});
      step(k8 + 7, std::integral_constant<int, 7>{});
    }
  } else {
    // ---- 4-byte elements: two steps per barrier, in two parts.
    //
    // Steps k and k + 1 (k even) together.  Before them the owners publish columns k and k + 1 and rows k and k + 1
    // as they are before step k.  What step k + 1 reads is column k + 1 and row k + 1 AFTER step k, and every thread
    // can work that out for its own rows and columns from what has been published:
    //   d[i][k+1] after step k = min(d[i][k+1], d[i][k] + d[k][k+1]),  d[k+1][j] after step k = min(d[k+1][j], d[k+1][k] + d[k][j])
    // (the sums and comparisons that step k itself makes for those elements, made again).  An element then takes
    // both steps' candidates in one 3-input minimum: three instructions per element and two steps instead of four,
    // and one round of publish / barrier / read-back per two steps.
    //
    // The steps depend on each other, and what lies between two pairs of them (publishing, the barrier, reading
    // back) would add its full latency to every pair.  So a pair is done in two parts:
    //   A. the patch's rows and columns (k + 2) & 7 and (k + 3) & 7 -- every thread's, since which thread owns
    //      rows / columns k + 2 and k + 3 is only known at run time -- then the owners publish them, then the barrier;
    //   B. the reads for the next pair are issued, and the other 36 elements are done while they are on their way.
    //
    // The published lines are what hist gets (for these element types hist holds, for odd k, column k and row k as
    // they are before step k - 1: fw_parents_block makes the same correction), copied from LDS by half the threads
    // a barrier after they were published.  There are four sets of lines in LDS, used in turn: a set is written again
    // three barriers after it was read for the last time.  (Nothing in this loop may wait for memory: stores
    // to hist are on their way all the time, and a wait for any load would wait for them.)
    const unsigned row_lds[4] = {lds(rowbuf + (0) * FW_BLOCK + 8 * tj), lds(rowbuf + (2) * FW_BLOCK + 8 * tj), lds(rowbuf + (4) * FW_BLOCK + 8 * tj), lds(rowbuf + (6) * FW_BLOCK + 8 * tj)};
    const unsigned col_lds[4] = {lds(colbuf + (0) * FW_BLOCK + 8 * ti), lds(colbuf + (2) * FW_BLOCK + 8 * ti), lds(colbuf + (4) * FW_BLOCK + 8 * ti), lds(colbuf + (6) * FW_BLOCK + 8 * ti)};
    // (the lines' addresses in vector registers of the thread's own: as values that are the same for all
    // threads the compiler fetches them again for every pair, and waits for that with the reads above)
    unsigned row_at_0 = lds(rowbuf), col_at_0 = lds(colbuf);
    asm volatile("" : "+v"(row_at_0), "+v"(col_at_0));
    struct Lines {
      T c0[8], c1[8], r0[8], r1[8];  // columns k, k + 1 at my rows, rows k, k + 1 at my columns, before step k
      T at_01, at_10;                // d[k][k + 1], d[k + 1][k]
    };
    auto publish = [&](int kn, auto setc, auto sc) {
      constexpr int SET = decltype(setc)::value, S = decltype(sc)::value;
      if ((kn >> 3) == ti) {  // my patch holds rows kn and kn + 1
        put_row(row_lds[SET], std::integral_constant<int, S>{}, std::integral_constant<int, 0>{});
        put_row(row_lds[SET], std::integral_constant<int, S + 1>{}, std::integral_constant<int, FW_BLOCK>{});
      }
      if ((kn >> 3) == tj) {  // my patch holds columns kn and kn + 1
        put_col(col_lds[SET], std::integral_constant<int, S>{}, std::integral_constant<int, 0>{});
        put_col(col_lds[SET], std::integral_constant<int, S + 1>{}, std::integral_constant<int, FW_BLOCK>{});
      }
      // (the barrier that follows is the compiler's, which does not know of the instructions above)
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    };
    auto fetch = [&](Lines &l, int set, int kn) {
      get8(l.c0, colbuf + (2 * set) * FW_BLOCK + 8 * ti);
      get8(l.c1, colbuf + (2 * set + 1) * FW_BLOCK + 8 * ti);
      get8(l.r0, rowbuf + (2 * set) * FW_BLOCK + 8 * tj);
      get8(l.r1, rowbuf + (2 * set + 1) * FW_BLOCK + 8 * tj);
      const unsigned at = unsigned(((2 * set) * FW_BLOCK + ((kn + 1) & (FW_BLOCK - 1))) * sizeof(T));
      l.at_01 = *(const LT *)(size_t)(row_at_0 + at);
      l.at_10 = *(const LT *)(size_t)(col_at_0 + at);
    };
    // the four lines of a set (steps kn and kn + 1) from LDS to hist: 16 bytes per thread of the first two waves
    const int line = tid >> 5, piece = 4 * (tid & 31);
    GT *const hist_line = (line < 2 ? hist_col : hist_row) + (line & 1) * FW_BLOCK + piece;
    auto keep = [&](int set, int kn) {
      if (tid < 128 && kn < FW_BLOCK)
        *reinterpret_cast<GV4 *>(hist_line + kn * FW_BLOCK) =
            *(const LV4 *)(size_t)((line < 2 ? col_at_0 : row_at_0) + unsigned(((2 * set + (line & 1)) * FW_BLOCK + piece) * sizeof(T)));
    };
    Lines cur_l;
    auto pair = [&](int k, auto uc) {
      constexpr int U = decltype(uc)::value;  // k & 7: 0, 2, 4, 6
      constexpr int N = (U + 2) & 7;          // the rows and columns N, N + 1 of the patch are what steps k + 2, k + 3 may need
      constexpr int O[6] = {N > 0 ? 0 : 2, N > 0 ? 1 : 3, N > 2 ? 2 : 4, N > 2 ? 3 : 5, N > 4 ? 4 : 6, N > 4 ? 5 : 7};
      constexpr int SET = U >> 1;
      Lines &l = cur_l;
      // column k + 1 and row k + 1 after step k
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        relax(l.c1[x], l.c0[x] + l.at_01);
        relax(l.r1[x], l.at_10 + l.r0[x]);
      }
      auto both = [&](auto ac, auto bc) {
        constexpr int A = decltype(ac)::value, B = decltype(bc)::value;
        relax2(cur[A][B], l.c0[A] + l.r0[B], l.c1[A] + l.r1[B]);
      };
      // A.
      static_for<8>([&](auto bc) {
        both(std::integral_constant<int, N>{}, bc);
        both(std::integral_constant<int, N + 1>{}, bc);
      });
      static_for<6>([&](auto ic) {
        both(std::integral_constant<int, O[decltype(ic)::value]>{}, std::integral_constant<int, N>{});
        both(std::integral_constant<int, O[decltype(ic)::value]>{}, std::integral_constant<int, N + 1>{});
      });
      __builtin_amdgcn_sched_barrier(0);
      publish(k + 2, std::integral_constant<int, (SET + 1) & 3>{}, std::integral_constant<int, N>{});
      __syncthreads();
      Lines next;
      fetch(next, (SET + 1) & 3, k + 2);
      __builtin_amdgcn_sched_barrier(0);
      // B.
      static_for<6>([&](auto ic) {
        static_for<6>([&](auto jc) {
          both(std::integral_constant<int, O[decltype(ic)::value]>{}, std::integral_constant<int, O[decltype(jc)::value]>{});
        });
      });
      __builtin_amdgcn_sched_barrier(0);
      keep((SET + 1) & 3, k + 2);
      cur_l = next;
    };
    publish(0, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});
    __syncthreads();
    fetch(cur_l, 0, 0);
    keep(0, 0);
    // steps beyond bb (up to the next multiple of eight) read rows and columns of the padding, which hold
    // +infinity and improve nothing
#pragma unroll 1
    for (int k8 = 0; k8 < bb; k8 += 8) {
      pair(k8 + 0, std::integral_constant<int, 0>{});
      pair(k8 + 2, std::integral_constant<int, 2>{});
      pair(k8 + 4, std::integral_constant<int, 4>{});
      pair(k8 + 6, std::integral_constant<int, 6>{});
    }
  }
#pragma unroll
  for (int b = 0; b < 8; ++b)
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      const int i = 8 * ti + a, j = 8 * tj + b;
      T v = cur[a][b];
      asm volatile("" : "+v"(v));  // (a value of its own: see the stores of init above)
      if (i < bb && j < bb) d[i + int64_t(j) * ld] = v;
    }
  return true;
}

// The same closure for a block that holds a -0: comparison and select, one step per barrier, and the block's rows and
// columns handed from step to step through the block itself in device memory (every thread stores what it lowered,
// and reads column k and row k from there), with the step loop rolled.  Two to three times slower than the form
// above, a fraction of its code, and nothing of it in scratch memory -- a form like the one above with comparisons
// keeps 64 comparison masks and as many candidates alive and spills hundreds of registers, which every workgroup
// of the kernel pays for in scratch space, whether it ever sees a -0 or not.
template <typename T>
__device__ __attribute__((noinline)) void fw_close_dist_exact(T *d_anywhere, int64_t ld, int bb, T *hist_anywhere) {
  typedef __attribute__((address_space(1))) T GT;
  GT *const d = (GT *)d_anywhere, *const hist = (GT *)hist_anywhere;
  GT *hist_col = hist, *hist_row = hist + FW_BLOCK * FW_BLOCK, *init = hist + 2 * FW_BLOCK * FW_BLOCK;
  const int tid = threadIdx.x & 255, ti = tid & 15, tj = tid >> 4;  // rows 8 ti .. 8 ti + 7, columns 8 tj .. 8 tj + 7
  const T inf = std::numeric_limits<T>::infinity();
  // (rows and columns of the padding are computed on the block's last row / column and never stored)
  int ic[8];
#pragma unroll
  for (int a = 0; a < 8; ++a) ic[a] = min(8 * ti + a, bb - 1);
  T cur[8][8];
#pragma unroll
  for (int b = 0; b < 8; ++b) {
    const GT *column = d + int64_t(min(8 * tj + b, bb - 1)) * ld;
#pragma unroll
    for (int a = 0; a < 8; ++a) {
      cur[a][b] = (8 * ti + a < bb && 8 * tj + b < bb) ? column[ic[a]] : inf;
      init[(8 * a + b) * 256 + tid] = cur[a][b];
    }
  }
  // what hist holds for 4-byte elements (fw_parents_block): for odd k column k and row k as before step k - 1
  constexpr int PAIRED = sizeof(T) == 4 ? 1 : 0;
#pragma unroll 1
  for (int k = 0; k < bb; ++k) {
    __syncthreads();  // what step k - 1 lowered is in the block
    T ci[8], rj[8];
#pragma unroll
    for (int a = 0; a < 8; ++a) ci[a] = d[ic[a] + int64_t(k) * ld];
#pragma unroll
    for (int b = 0; b < 8; ++b) rj[b] = d[k + int64_t(min(8 * tj + b, bb - 1)) * ld];
    if (!PAIRED || !(k & 1)) {
      const int lines = PAIRED ? 2 : 1;
      for (int q = 0; q < lines; ++q) {
        const int kq = min(k + q, bb - 1);
        if (tj == 0)
#pragma unroll
          for (int a = 0; a < 8; ++a) hist_col[(k + q) * FW_BLOCK + 8 * ti + a] = 8 * ti + a < bb ? (q ? T(d[ic[a] + int64_t(kq) * ld]) : ci[a]) : inf;
        if (ti == 0)
#pragma unroll
          for (int b = 0; b < 8; ++b)
            hist_row[(k + q) * FW_BLOCK + 8 * tj + b] = 8 * tj + b < bb ? (q ? T(d[kq + int64_t(min(8 * tj + b, bb - 1)) * ld]) : rj[b]) : inf;
      }
    }
    __syncthreads();  // everybody has read column k and row k (and k + 1) before anybody stores
#pragma unroll
    for (int b = 0; b < 8; ++b)
#pragma unroll
      for (int a = 0; a < 8; ++a) {
        const T cand = ci[a] + rj[b];
        if (cand < cur[a][b]) {
          cur[a][b] = cand;
          if (8 * ti + a < bb && 8 * tj + b < bb) d[8 * ti + a + int64_t(8 * tj + b) * ld] = cand;
        }
      }
  }
}

template <typename T>
__device__ __forceinline__ void fw_close_dist(T *d, int64_t ld, int bb, T *hist) {
  typedef __attribute__((address_space(3))) T LT;
  constexpr int LINES = sizeof(T) == 4 ? 8 : 4;
  __shared__ __attribute__((aligned(32))) T colbuf[LINES * FW_BLOCK], rowbuf[LINES * FW_BLOCK];
  if (!fw_close_dist_fast<T>(d, ld, bb, hist, (LT *)colbuf, (LT *)rowbuf)) fw_close_dist_exact<T>(d, ld, bb, hist);
}

// The predecessors of a diagonal block whose distances fw_close_dist has closed: workgroup b of 64 (256 threads)
// takes rows 64 (b & 1) .. + 63 and columns 4 (b >> 1) .. + 3, one element per thread, and runs the literal scan
// over the recorded columns and rows.  Only predecessors are written: the distances are those already there.
// For 4-byte elements hist holds, for odd k, column k and row k as they are before step k - 1; step k - 1's
// update of them is made here as fw_close_dist makes it (with the comparison: it never differs from the minimum
// on a block without -0, and a block with one was closed with the comparison).
template <typename T>
__device__ __forceinline__ void fw_parents_block(const T *hist, int32_t *parent, int64_t ldp, int bb, int k_base, int b) {
  const int row = (b & 1) * 64 + (threadIdx.x & 63);
  const int col = __builtin_amdgcn_readfirstlane((b >> 1) * 4 + (threadIdx.x >> 6));
  if (row >= bb || col >= bb) return;
  const T *hist_row = hist + FW_BLOCK * FW_BLOCK;
  const T *hc = hist + row, *hr = hist_row + col;
  T curr = hist[2 * FW_BLOCK * FW_BLOCK + (8 * (row & 7) + (col & 7)) * 256 + (row >> 3) + 16 * (col >> 3)];
  int32_t p = -1;
  auto scan = [&](const T prod, int k) {
    const bool lower = prod < curr;
    curr = pick(lower, prod, curr);
    p = lower ? k : p;
  };
  if constexpr (sizeof(T) == 4) {
    auto steps = [&](const T c0, T c1, const T r0, T r1, const T at_01, const T at_10, int k) {
      scan(c0 + r0, k);
      const T via_c = c0 + at_01, via_r = at_10 + r0;
      c1 = pick(via_c < c1, via_c, c1);
      r1 = pick(via_r < r1, via_r, r1);
      if (k + 1 < bb) scan(c1 + r1, k + 1);
    };
    int k = 0;
    for (; k + 16 <= bb; k += 16) {  // sixteen k at a time, their operands requested together
      T cv[16], rv[16], at_01[8], at_10[8];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        cv[u] = hc[(k + u) * FW_BLOCK];
        rv[u] = hr[(k + u) * FW_BLOCK];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        at_01[u] = hist_row[(k + 2 * u) * FW_BLOCK + k + 2 * u + 1];
        at_10[u] = hist[(k + 2 * u) * FW_BLOCK + k + 2 * u + 1];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) steps(cv[2 * u], cv[2 * u + 1], rv[2 * u], rv[2 * u + 1], at_01[u], at_10[u], k + 2 * u);
    }
    for (; k < bb; k += 2)
      steps(hc[k * FW_BLOCK], hc[(k + 1) * FW_BLOCK], hr[k * FW_BLOCK], hr[(k + 1) * FW_BLOCK], hist_row[k * FW_BLOCK + k + 1],
            hist[k * FW_BLOCK + k + 1], k);
  } else {
    int k = 0;
    for (; k + 16 <= bb; k += 16) {  // sixteen k at a time, their operands requested together
      T cv[16], rv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        cv[u] = hc[(k + u) * FW_BLOCK];
        rv[u] = hr[(k + u) * FW_BLOCK];
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) scan(cv[u] + rv[u], k + u);
    }
    for (; k < bb; ++k) scan(hc[k * FW_BLOCK] + hr[k * FW_BLOCK], k);
  }
  if (p >= 0) parent[row + int64_t(col) * ldp] = k_base + p;
}

template <typename T>
__global__ void __launch_bounds__(256) fw_parents_kernel(const T *hist, int32_t *parent, int64_t ldp, int bb, int k_base) {
  fw_parents_block<T>(hist, parent, ldp, bb, k_base, blockIdx.x);
}
constexpr int FW_PARENT_BLOCKS = (FW_BLOCK / 64) * (FW_BLOCK / 4);

// two independent products in one launch (the block row and the block column of a blocked
// Floyd-Warshall step, each too small to fill the chip): after the first FW_PARENT_BLOCKS workgroups, which
// with hist set find the predecessors of the diagonal block at k_base (closed by fw_close_dist in the launch
// before) and otherwise have nothing to do, the next blocks0 workgroups work on g0, the others on g1
template <typename T>
__global__ void __launch_bounds__(256) fwgemm_pair_kernel(FwArgs g0, FwArgs g1, int blocks0, const T *hist, int32_t *hist_parent,
                                                          int64_t ldp, int hist_bb, int k_base) {
  int b = blockIdx.x;
  if (b < FW_PARENT_BLOCKS) {
    if (hist) fw_parents_block<T>(hist, hist_parent, ldp, hist_bb, k_base, b);
    return;
  }
  b -= FW_PARENT_BLOCKS;
  if (b < blocks0) {
    const int gx = (g0.m + 63) / 64;
    fwgemm_rowcols_block<T>(g0, b % gx, b / gx);
  } else {
    const int gx = (g1.m + 63) / 64;
    fwgemm_rowcols_block<T>(g1, (b - blocks0) % gx, (b - blocks0) / gx);
  }
}

// The tile kernel.  Grid (tiles along m, tiles along n); with g.ahead_bb > 0 the grid has one more row,
// whose first workgroup -- the first one the launch starts -- closes the next block step's diagonal
// block while the workgroups of the other rows do the product's tiles, all but that block.  The block's
// 128 dependent steps take about as long as the whole product and nothing else of the next block step can
// start before them; here they cost one of the launch's 512 places.  Only where a tile is a whole
// diagonal block (4-byte elements; the host asks for nothing else).
template <typename T, int TM, int TN, int SN, int BK, bool GUARD, bool HAS_AT>
__global__ void __launch_bounds__(256, 2) fwgemm_tile_kernel(FwArgs g) {
  constexpr int BM = 16 * TM, BN = 16 * TN;
  constexpr bool CAN_CLOSE = FW_BLOCK % BM == 0 && FW_BLOCK % BN == 0;
  int bx = blockIdx.x, by = blockIdx.y;
  if constexpr (CAN_CLOSE) {
    if (g.ahead_bb > 0) {
      if (by == 0) {
        // Which workgroup of the extra row closes the block: workgroups go to the chip's eight dies in turn, by
        // their number in the launch, and a die starts them in order as places come free.  The closure holds
        // its place for most of the launch, so it goes to the die that has the least to do: with a number of
        // tile columns that is a multiple of eight, the tiles of the skipped rows -- which return at once --
        // all have numbers that are bx modulo eight.  (On any other die the last tile waits for the
        // closure's place and the launch ends 15 us later.)
        const int closer = (gridDim.x % 8 == 0 && g.skip_r1 > g.skip_r0) ? (g.skip_r0 / BM) % 8 : 0;
        if (bx == closer)
          fw_close_dist<T>(static_cast<T *>(g.dist) + g.ahead0 + int64_t(g.ahead0) * g.ldc, g.ldc, g.ahead_bb,
                           static_cast<T *>(g.hist));
        return;
      }
      by -= 1;
      const int r0 = bx * BM - g.ahead0, c0 = by * BN - g.ahead0;
      if (r0 >= 0 && r0 < FW_BLOCK && c0 >= 0 && c0 < FW_BLOCK) return;
    }
  }
  fwgemm_tile_body<T, TM, TN, SN, BK, GUARD, HAS_AT>(g, bx, by);
}

// ---- the predecessor-tracking product on the hand-scheduled direct-to-LDS tile (direct_tile.h, direct_asm.h)
//
// For whole, aligned fp32 problems with the k-contiguous image of A at hand.  Column-major dist = A (x) B is the
// row-major transposed problem dist^T = B^T (x) A^T, so the tile's "A" panel is B (k-contiguous) and its "B" panel
// is A (x-contiguous): the generated loop's kx form, 512 threads, 256 columns x 128 rows of dist per workgroup, the
// loop's accumulators being the running minima themselves (they start from dist).  What the loop cannot do is
// remember WHEN a minimum improved, and its 128 registers leave no room for that; so this kernel runs it with
// 256 registers (two waves per SIMD) and keeps, beside it, a copy of the accumulators as they were two k-tiles
// ago and a 16-bit chunk index per element: after every second k-tile "accumulator < copy" (strict) records
// the chunk of 32 k, four instructions per element and 32 k against the 48 of the terms themselves.  The
// epilogue is the tile kernel's: improved elements are queued in LDS and looked up, 32 values of A's row (from
// the k-contiguous image) and 32 of B's column each, first k whose sum equals the minimum.
constexpr int FWD_CHUNK = 32;
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) fwgemm_direct_kernel(FwArgs g) {
  typedef DirectTile<float, kMinimum, kPlus, true, false, 32, 16> Tile;
  typedef AsmLoop<float, kMinimum, kPlus, true, false>::type Loop;
  typedef vec4_of<float>::type V4;
  constexpr int BC = 256, BR = 128, BK = 16, STAGES = 3;   // dist columns and rows per workgroup
  __shared__ Tile::Smem sm;
  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16, lane = tid & 63, wave = tid >> 6;
  int bc, br;
  Tile::tile_coords(blockIdx.x, g.n / BC, g.m / BR, bc, br);
  const int n0 = bc * BC, m0 = br * BR;
  const float *A = static_cast<const float *>(g.A);
  const float *B = static_cast<const float *>(g.B);
  float *dist = static_cast<float *>(g.dist);
  // output (i, j) of the thread: dist column n0 + 32 i + ty, dist row m0 + 64 (j / 4) + 4 tx + j % 4
  auto col_of = [&](int i) { return n0 + 32 * i + ty; };
  auto row_of = [&](int j) { return m0 + 64 * (j >> 2) + 4 * tx + (j & 3); };

  AsmRegs r;
  // element e = 8 i + j: the loop's accumulator is v(e); its value before the chunk in hand run[e / 16][e % 16] =
  // v(128 + e); its chunk index 16 bits of chunk[e / 32][(e / 2) % 16] = v(192 + e / 2), 0xffff = never improved
  asm_v16 run[4], chunk[2];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const V4 v = *reinterpret_cast<const V4 *>(dist + row_of(4 * h) + int64_t(col_of(i)) * g.ldc);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        run[i >> 1][(i & 1) * 8 + 4 * h + e] = v[e];
        r.acc[i >> 1][(i & 1) * 8 + 4 * h + e] = v[e];
      }
    }
  }
#pragma unroll
  for (int v = 0; v < 2; ++v) chunk[v] = asm_v16(__builtin_bit_cast(float, 0xffffffffu));
#pragma unroll
  for (int v = 0; v < 3; ++v) r.frag[v] = asm_v16(0.0f);

  // global -> LDS: the tile's "A" panel is B's 256 columns (k-contiguous, two pieces per wave and k-tile), its
  // "B" panel A's 128 rows (x-contiguous, one piece per wave)
  const char *base_a = reinterpret_cast<const char *>(B + int64_t(n0) * g.ldb);
  const char *base_b = reinterpret_cast<const char *>(A + m0);
  const long long a_next = (long long)BK * 4, b_next = (long long)BK * g.lda * 4;
  const unsigned b_kbytes = (unsigned)g.lda * 4u;
  const unsigned off_a0 = Tile::tile_offset<true, BC>((wave * 2 + 0) * 64 + lane, Tile::x_offset<true, BC>((wave * 2 + 0) * 64 + lane, g.ldb, n0, g.n), 4u, BK);
  const unsigned off_a1 = Tile::tile_offset<true, BC>((wave * 2 + 1) * 64 + lane, Tile::x_offset<true, BC>((wave * 2 + 1) * 64 + lane, g.ldb, n0, g.n), 4u, BK);
  const unsigned off_b0 = Tile::tile_offset<false, BR>(wave * 64 + lane, Tile::x_offset<false, BR>(wave * 64 + lane, 1, m0, g.m), b_kbytes, BK);
  auto fetch = [&](int stage) {
    Tile::dma16(reinterpret_cast<const float *>(base_a + off_a0), &sm.a[stage][(wave * 2 + 0) * 256]);
    Tile::dma16(reinterpret_cast<const float *>(base_a + off_a1), &sm.a[stage][(wave * 2 + 1) * 256]);
    Tile::dma16(reinterpret_cast<const float *>(base_b + off_b0), &sm.b[stage][wave * 256]);
    base_a += a_next;
    base_b += b_next;
  };
  const int ntiles = g.k / BK;   // the host sends whole pairs of k-tiles only
  fetch(0);
  __syncthreads();
  fetch(1);  // from here base_a / base_b point at tile 2
  const unsigned m0_a0 = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) float *)&sm.a[0][(wave * 2) * 256]);
  const unsigned m0_b0 = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) float *)&sm.b[0][wave * 256]);
  constexpr unsigned A_STAGE = BK * BC * 4, B_STAGE = BK * BR * 4;
  unsigned a_addr = (unsigned)(size_t)(__attribute__((address_space(3))) float *)&sm.a[0][0] + ty * 16;
  unsigned b_addr = (unsigned)(size_t)(__attribute__((address_space(3))) float *)&sm.b[0][0] + tx * 16;
  Loop::prime(r, a_addr, b_addr);
  int stage = 0;
  auto one_tile = [&](int t) {
    const int next = stage + 1 == STAGES ? 0 : stage + 1, stage2 = next + 1 == STAGES ? 0 : next + 1;
    Loop::tile(r, a_addr, b_addr, (unsigned)((next - stage) * (int)A_STAGE), (unsigned)((next - stage) * (int)B_STAGE),
               ntiles - (t + 2), m0_a0 + stage2 * A_STAGE, m0_b0 + stage2 * B_STAGE, off_a0, off_a1, off_b0, base_a, base_b);
    base_a += a_next;
    base_b += b_next;
    stage = next;
  };
#pragma unroll 1
  for (int t = 0; t < ntiles; t += 2) {   // a chunk of 32 k: two k-tiles, then the bookkeeping (no branch around it)
    one_tile(t);
    one_tile(t + 1);
    // the bookkeeping (gen/fwgemm_merge.inc, written by gen_direct_asm.py): a cheap test whether any of the
    // wave's elements changed in this chunk, and only then, per element, "now < before" => chunk index, before = now
    const uint32_t c = (uint32_t)(t >> 1);
    asm volatile(
#include "gen/fwgemm_merge.inc"
        : "+{v[0:15]}"(r.acc[0]), "+{v[16:31]}"(r.acc[1]), "+{v[32:47]}"(r.acc[2]), "+{v[48:63]}"(r.acc[3]),
          "+{v[128:143]}"(run[0]), "+{v[144:159]}"(run[1]), "+{v[160:175]}"(run[2]), "+{v[176:191]}"(run[3]),
          "+{v[192:207]}"(chunk[0]), "+{v[208:223]}"(chunk[1])
        : [chunk] "v"(c)
        : "v224", "vcc");
  }

  // ---- improved elements: the first k of the recorded chunk whose sum equals the minimum.  As many whole canonical
  // rows i (one dist column per thread each) of the lanes' outputs as fit go into a queue in LDS (the panels are done
  // with; one row, at most 512 x 8 elements, always fits), which all 512 threads then work off (lookup_queue).
  constexpr int CAP = sizeof(Tile::Smem) / 8 / 512 * 512;
  static_assert(CAP >= 512 * 8, "a row of the lanes' outputs must fit in the panels");
  // Where an element goes in the queue follows from counts alone, without a shared counter: row by row, inside a
  // row wave by wave, inside a wave output j by output j, inside an output lane by lane.
  __shared__ int wave_count[8][8];
  uint32_t *q_code = reinterpret_cast<uint32_t *>(&sm.a[0][0]);   // row | column << 7 | chunk << 15, inside the tile
  float *q_want = reinterpret_cast<float *>(q_code + CAP);
  int tx2 = tx, ty2 = ty;
  asm volatile("" : "+v"(tx2), "+v"(ty2));
  auto chunk_of = [&](auto ic, auto jc) -> uint32_t {
    constexpr int I = decltype(ic)::value, J = decltype(jc)::value;
    const uint32_t w = __builtin_bit_cast(uint32_t, (float)chunk[I >> 2][(I & 3) * 4 + (J >> 1)]);
    return (J & 1) ? w >> 16 : w & 0xffffu;
  };
  __syncthreads();  // everybody is done with the panels
  static_for<8>([&](auto ic) {
    constexpr int I = decltype(ic)::value;
    int n_improved = 0;  // in this row, over the wave
    static_for<8>([&](auto jc) { n_improved += __builtin_popcountll(__builtin_amdgcn_ballot_w64(chunk_of(ic, jc) != 0xffffu)); });
    if (lane == 0) wave_count[wave][I] = n_improved;
  });
  __syncthreads();
  int before_me[8], row_count[8];  // improved elements of the row in the waves before mine / in all waves
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    before_me[i] = row_count[i] = 0;
#pragma unroll
    for (int w = 0; w < 8; ++w) {
      const int n = __builtin_amdgcn_readfirstlane(wave_count[w][i]);
      before_me[i] += w < wave ? n : 0;
      row_count[i] += n;
    }
  }
  for (int i0 = 0; i0 < 8;) {  // (the same for every thread)
    int total = 0, i1 = i0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {  // as many whole rows from i0 on as fit
      if (i < i0 || i != i1) continue;
      if (i > i0 && total + row_count[i] > CAP) continue;
      total += row_count[i];
      i1 = i + 1;
    }
    if (total > 0) {
      int base = 0;  // of the row in the queue
      static_for<8>([&](auto ic) {
        constexpr int I = decltype(ic)::value;
        if (I < i0 || I >= i1) return;
        int slot0 = base + before_me[I];  // of my wave's next output of this row
        static_for<8>([&](auto jc) {
          constexpr int J = decltype(jc)::value;
          const uint32_t ch = chunk_of(ic, jc);
          const unsigned long long improved = __builtin_amdgcn_ballot_w64(ch != 0xffffu);
          if (ch != 0xffffu) {
            const int slot = slot0 + __builtin_amdgcn_mbcnt_hi(uint32_t(improved >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(improved), 0u));
            q_code[slot] = uint32_t(64 * (J >> 2) + 4 * tx2 + (J & 3)) | uint32_t(32 * I + ty2) << 7 | ch << 15;
            q_want[slot] = run[I >> 1][(I & 1) * 8 + J];
          }
          slot0 += __builtin_popcountll(improved);
        });
        base += row_count[I];
      });
      __syncthreads();
      lookup_queue<float, 512, FWD_CHUNK, true, 7, 8>(g, q_code, q_want, total, tid, m0, n0);
      __syncthreads();  // the queue is free again
    }
    i0 = i1;
  }
}

// whole tiles of 128 rows x 256 columns, k in whole chunks, every operand (and the k-contiguous image of A)
// 16-byte aligned with leading dimensions that are multiples of 4, no rows / columns to skip, chunk indices in 16 bits
bool fwgemm_direct_ok(const FwArgs &g) {
  auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  if (g.m <= 0 || g.n <= 0 || g.k < 2 * FWD_CHUNK || g.m % 128 || g.n % 256 || g.k % FWD_CHUNK || g.k / FWD_CHUNK >= 0xffff) return false;
  if (!g.At || !al(g.A) || !al(g.B) || !al(g.dist) || !al(g.At)) return false;
  if (g.lda % 4 || g.ldb % 4 || g.ldc % 4 || g.ldat % 4) return false;
  if (g.skip_r1 > g.skip_r0 || g.skip_c1 > g.skip_c0 || g.ahead_bb > 0 || g.out_t) return false;
  // 32-bit byte offsets inside a tile
  if (int64_t(g.ldb) * 256 * 4 >= (int64_t(1) << 31) || int64_t(g.lda) * 16 * 4 >= (int64_t(1) << 31)) return false;
  return int64_t(g.m / 128) * (g.n / 256) <= 0x7fffffff;
}

template <typename T, int TM, int TN, int SN, int BK>
hipError_t launch_tile(const FwArgs &g, hipStream_t stream) {
  constexpr int BM = 16 * TM, BN = 16 * TN;
  // (the unguarded form queues improved elements with their chunk of BK k-values in 18 bits)
  const bool whole = g.m % BM == 0 && g.n % BN == 0 && g.k % BK == 0 && g.k < (1 << 22);
  const size_t vec = 4 * sizeof(T);
  const bool aligned = reinterpret_cast<uintptr_t>(g.A) % vec == 0 && reinterpret_cast<uintptr_t>(g.B) % vec == 0 &&
                       g.lda % 4 == 0 && g.ldb % 4 == 0;
  if (g.ahead_bb > 0 && (FW_BLOCK % BM || FW_BLOCK % BN)) return hipErrorInvalidValue;
  dim3 grid((g.m + BM - 1) / BM, (g.n + BN - 1) / BN + (g.ahead_bb > 0 ? 1 : 0));
  if (g.At) {
    const bool at_aligned = reinterpret_cast<uintptr_t>(g.At) % vec == 0 && g.ldat % 4 == 0;
    if (whole && aligned && at_aligned)
      launch_kernel((fwgemm_tile_kernel<T, TM, TN, SN, BK, false, true>), grid, dim3(256), 0, stream, g);
    else
      launch_kernel((fwgemm_tile_kernel<T, TM, TN, SN, BK, true, true>), grid, dim3(256), 0, stream, g);
  } else if (whole && aligned) {
    launch_kernel((fwgemm_tile_kernel<T, TM, TN, SN, BK, false, false>), grid, dim3(256), 0, stream, g);
  } else {
    launch_kernel((fwgemm_tile_kernel<T, TM, TN, SN, BK, true, false>), grid, dim3(256), 0, stream, g);
  }
  return take_launch_status();
}

// src (rows x cols, column-major, leading dimension ld) -> w, a column-major copy with leading
// dimension ldw, and wt, its transpose (wt[c + r * ldwt] = src[r, c]), in one pass over
// 64 x 64 blocks; either destination may be null
template <typename T>
__global__ void __launch_bounds__(256) snapshot_kernel(const T *src, int64_t ld, T *w, int64_t ldw, T *wt, int64_t ldwt,
                                                       int rows, int cols) {
  __shared__ T tile[64][65];
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int j = ty; j < 64; j += 4) {
    const int r = r0 + tx, c = c0 + j;
    if (r < rows && c < cols) {
      const T v = src[r + int64_t(c) * ld];
      if (w) w[r + int64_t(c) * ldw] = v;
      tile[j][tx] = v;
    }
  }
  if (!wt) return;
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols) wt[c + int64_t(r) * ldwt] = tile[tx][i];
  }
}

template <typename T>
hipError_t snapshot(const void *src, int64_t ld, void *w, int64_t ldw, void *wt, int64_t ldwt, int rows, int cols,
                    hipStream_t s) {
  const dim3 grid((rows + 63) / 64, (cols + 63) / 64);
  launch_kernel(snapshot_kernel<T>, grid, dim3(256), 0, s, static_cast<const T *>(src), ld, static_cast<T *>(w), ldw,
                     static_cast<T *>(wt), ldwt, rows, cols);
  return take_launch_status();
}

// two copies in one launch: the first blocks0 workgroups copy (src0 -> w0), the others (src1 -> w1)
template <typename T>
__global__ void __launch_bounds__(256) snapshot_pair_kernel(const T *src0, T *w0, int64_t ldw0, int rows0, int cols0,
                                                            const T *src1, T *w1, int64_t ldw1, int rows1, int cols1,
                                                            int64_t ld, int blocks0) {
  int b = blockIdx.x;
  const bool first = b < blocks0;
  if (!first) b -= blocks0;
  const T *src = first ? src0 : src1;
  T *w = first ? w0 : w1;
  const int64_t ldw = first ? ldw0 : ldw1;
  const int rows = first ? rows0 : rows1, cols = first ? cols0 : cols1;
  const int gx = (rows + 63) / 64;
  const int r = (b % gx) * 64 + (threadIdx.x & 63), c0 = (b / gx) * 64 + (threadIdx.x >> 6);
  if (r >= rows) return;
  // (all of a thread's 16 loads, then its stores: source and copy may be the same memory for all the compiler
  // knows, and one load after each store is sixteen trips to memory in a row)
  T v[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) v[u] = src[r + int64_t(min(c0 + 4 * u, cols - 1)) * ld];
#pragma unroll
  for (int u = 0; u < 16; ++u)
    if (c0 + 4 * u < cols) w[r + int64_t(c0 + 4 * u) * ldw] = v[u];
}

// Floyd-Warshall inside one diagonal block of at most FW_BLOCK x FW_BLOCK: k ascending,
// d[i][j] > d[i][k] + d[k][j] => d[i][j] = the sum, parent = k_base + k.  One workgroup of 1024
// threads holds the block in registers, a 4 x 4 patch per thread.  Step k needs column k and row k
// only, and they do not change during step k (the block's diagonal is not negative): every step
// reads them from two 128-element LDS buffers and publishes column k + 1 and row k + 1 into the
// other pair, so one barrier per step is enough and a thread reads two vectors per 16 updates.
template <typename T>
__global__ void __launch_bounds__(1024) fw_diagonal_kernel(T *d, int64_t ld, int32_t *parent, int64_t ldp, int bb, int k_base) {
  typedef typename vec4_of<T>::type V4;
  __shared__ __attribute__((aligned(32))) T colbuf[2][FW_BLOCK];  // d[i][k] for the step that reads this buffer
  __shared__ __attribute__((aligned(32))) T rowbuf[2][FW_BLOCK];  // d[k][j]
  const int ti = threadIdx.x & 31, tj = threadIdx.x >> 5;  // rows 4 ti .. 4 ti + 3, columns 4 tj .. 4 tj + 3
  const T inf = std::numeric_limits<T>::infinity();
  T cur[4][4];  // [row in patch][column in patch]
  int32_t par[4][4];
#pragma unroll
  for (int b = 0; b < 4; ++b)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int i = 4 * ti + a, j = 4 * tj + b;
      cur[a][b] = (i < bb && j < bb) ? d[i + int64_t(j) * ld] : inf;
      par[a][b] = -1;
    }
  // S = kn & 3, the row / column of the patch that is published, is a compile-time constant
  // (the step loop is unrolled by four): indexed by a run-time value the patch would be
  // moved to scratch memory, and every step would wait for memory
  auto publish = [&](int kn, int buf, auto sc) {
    constexpr int S = decltype(sc)::value;
    if ((kn >> 2) == ti) {  // my patch holds row kn
      V4 v;
#pragma unroll
      for (int b = 0; b < 4; ++b) v[b] = cur[S][b];
      *reinterpret_cast<V4 *>(&rowbuf[buf][4 * tj]) = v;
    }
    if ((kn >> 2) == tj) {  // my patch holds column kn
      V4 v;
#pragma unroll
      for (int a = 0; a < 4; ++a) v[a] = cur[a][S];
      *reinterpret_cast<V4 *>(&colbuf[buf][4 * ti]) = v;
    }
  };
  auto step = [&](int k, auto uc) {
    constexpr int U = decltype(uc)::value;  // k & 3
    const int buf = U & 1;
    const V4 ci = *reinterpret_cast<const V4 *>(&colbuf[buf][4 * ti]);
    const V4 rj = *reinterpret_cast<const V4 *>(&rowbuf[buf][4 * tj]);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const T cand = ci[a] + rj[b];
        const bool lower = cand < cur[a][b];
        cur[a][b] = pick(lower, cand, cur[a][b]);
        par[a][b] = lower ? k_base + k : par[a][b];
      }
    // the other pair of buffers: nobody reads it before the barrier, and nobody is still
    // reading it from the step before (everybody has passed that step's barrier)
    publish(k + 1, buf ^ 1, std::integral_constant<int, (U + 1) & 3>{});
    __syncthreads();
  };
  publish(0, 0, std::integral_constant<int, 0>{});
  __syncthreads();
  // steps beyond bb (up to the next multiple of four) read rows and columns of the padding,
  // which hold +infinity and improve nothing
  for (int k4 = 0; k4 < bb; k4 += 4) {
    step(k4 + 0, std::integral_constant<int, 0>{});
    step(k4 + 1, std::integral_constant<int, 1>{});
    step(k4 + 2, std::integral_constant<int, 2>{});
    step(k4 + 3, std::integral_constant<int, 3>{});
  }
#pragma unroll
  for (int b = 0; b < 4; ++b)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int i = 4 * ti + a, j = 4 * tj + b;
      if (i < bb && j < bb && par[a][b] >= 0) {
        d[i + int64_t(j) * ld] = cur[a][b];
        parent[i + int64_t(j) * ldp] = par[a][b];
      }
    }
}

template <typename T> hipError_t launch_naive(const FwArgs &g, hipStream_t stream) {
  dim3 grid((g.m + 63) / 64, (g.n + 3) / 4);
  launch_kernel(fwgemm_naive_kernel<T>, grid, dim3(256), 0, stream, g);
  return take_launch_status();
}

int check(int dtype, int m, int n, int k, const void *A, int64_t lda, const void *B, int64_t ldb, const void *dist,
          int64_t ldc, const int32_t *parent, int64_t ldp, int kernel) {
  if (dtype != CUASR_AMD_F32 && dtype != CUASR_AMD_F64) return CUASR_AMD_ERROR_INVALID_DATA_TYPE;
  if (m < 0 || n < 0 || k < 0) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (lda < (m > 1 ? m : 1) || ldb < (k > 1 ? k : 1) || ldc < (m > 1 ? m : 1) || ldp < (m > 1 ? m : 1))
    return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (kernel != CUASR_AMD_KERNEL_AUTO && kernel != CUASR_AMD_KERNEL_NAIVE && kernel != CUASR_AMD_KERNEL_VALU)
    return CUASR_AMD_ERROR_NOT_SUPPORTED;
  if (m == 0 || n == 0) return CUASR_AMD_SUCCESS;
  if (!dist || !parent || (k > 0 && (!A || !B))) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  const size_t es = dtype == CUASR_AMD_F64 ? 8 : 4;
  if (reinterpret_cast<uintptr_t>(A) % es || reinterpret_cast<uintptr_t>(B) % es ||
      reinterpret_cast<uintptr_t>(dist) % es || reinterpret_cast<uintptr_t>(parent) % 4)
    return CUASR_AMD_ERROR_MISALIGNED_OPERAND;
  return CUASR_AMD_SUCCESS;
}

}  // namespace
}  // namespace cuasr_amd

using namespace cuasr_amd;

namespace {
struct FwExtra {
  const void *At = nullptr; int64_t ldat = 0;
  int k_base = 0, skip_r0 = 0, skip_r1 = 0, skip_c0 = 0, skip_c1 = 0;
  // blocked Floyd-Warshall: let the launch also close the diagonal block that starts at ahead0 (ahead_bb rows),
  // which the product then leaves alone.  Only the tile kernel can; *closed_ahead says whether this launch did.
  int ahead0 = 0, ahead_bb = 0;
  void *hist = nullptr;
  bool *closed_ahead = nullptr;
};
// one-thread-per-element kernel or tiles: a launch of a few workgroups is better spread over one thread per
// element, and so is one of few tiles (the tile kernel's workgroups would each run alone on a compute
// unit): measured on square problems, the two kernels meet at about 100 tiles (1024^3: 193 against 270 us,
// 1280^3: 356 against 334, 1408^3: 466 against 366)
bool takes_naive_kernel(int m, int n, int kernel) {
  const int64_t tiles = ((int64_t(m) + 127) / 128) * ((int64_t(n) + 127) / 128);
  const bool tiny = int64_t(m) * n < 64 * 64 || tiles < 96;
  return kernel == CUASR_AMD_KERNEL_NAIVE || (kernel == CUASR_AMD_KERNEL_AUTO && tiny);
}
int fwgemm_run(int dtype, int m, int n, int k, const void *A, int64_t lda, const void *B, int64_t ldb, void *dist,
               int64_t ldc, int32_t *parent, int64_t ldp, const FwExtra &x, int kernel, void *stream) {
  const int st = check(dtype, m, n, k, A, lda, B, ldb, dist, ldc, parent, ldp, kernel);
  if (st != CUASR_AMD_SUCCESS || m == 0 || n == 0 || k == 0) return st;
  FwArgs g{m, n, k, A, lda, B, ldb, dist, ldc, parent, ldp, x.At, x.ldat, x.k_base,
           x.skip_r0, x.skip_r1, x.skip_c0, x.skip_c1, nullptr, 0, 0, 0, nullptr};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool naive = takes_naive_kernel(m, n, kernel);
  if (!naive && x.ahead_bb > 0 && x.hist) {
    g.ahead0 = x.ahead0;
    g.ahead_bb = x.ahead_bb;
    g.hist = x.hist;
  }
  if (x.closed_ahead) *x.closed_ahead = g.ahead_bb > 0;
  hipError_t e;
  if (dtype == CUASR_AMD_F32 && !naive && kernel == CUASR_AMD_KERNEL_AUTO && fwgemm_direct_ok(g)) {
    launch_kernel(fwgemm_direct_kernel, dim3((unsigned)(int64_t(g.m / 128) * (g.n / 256))), dim3(512), 0, s, g);
    return take_launch_status() == hipSuccess ? CUASR_AMD_SUCCESS : CUASR_AMD_ERROR_INTERNAL;
  }
  if (dtype == CUASR_AMD_F32) e = naive ? launch_naive<float>(g, s) : launch_tile<float, 8, 8, 4, 16>(g, s);
  else e = naive ? launch_naive<double>(g, s) : launch_tile<double, 4, 8, 4, 16>(g, s);
  return e == hipSuccess ? CUASR_AMD_SUCCESS : CUASR_AMD_ERROR_INTERNAL;
}
}  // namespace

extern "C" int cuasr_amd_fwgemm(int dtype, int m, int n, int k, const void *A, int64_t lda, const void *B, int64_t ldb,
                                void *dist, int64_t ldc, int32_t *parent, int64_t ldp, int kernel, void *stream) {
  return fwgemm_run(dtype, m, n, k, A, lda, B, ldb, dist, ldc, parent, ldp, FwExtra{}, kernel, stream);
}

extern "C" size_t cuasr_amd_apsp_workspace_bytes(int dtype, int n) {
  if (n <= 0 || (dtype != CUASR_AMD_F32 && dtype != CUASR_AMD_F64)) return 0;
  return 2 * size_t(dtype == CUASR_AMD_F64 ? 8 : 4) * size_t(n) * size_t(n);  // the snapshot and its transpose
}

extern "C" int cuasr_amd_apsp_squaring(int dtype, int n, void *dist, int64_t ld, int32_t *parent, int64_t ldp,
                                       void *workspace, int iterations, void *stream) {
  const int64_t ldw = n > 0 ? n : 1;
  const int st = check(dtype, n, n, n, workspace, ldw, workspace, ldw, dist, ld, parent, ldp, CUASR_AMD_KERNEL_AUTO);
  if (n > 0 && !workspace) return CUASR_AMD_ERROR_WORKSPACE_NULL;
  if (st != CUASR_AMD_SUCCESS) return st;
  if (iterations < 0) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (n == 0) return CUASR_AMD_SUCCESS;
  if (iterations == 0)  // paths of up to n - 1 edges: ceil(log2(n - 1)) squarings
    for (int64_t reach = 1; reach < n - 1; reach *= 2) ++iterations;
  const size_t es = dtype == CUASR_AMD_F64 ? 8 : 4;
  hipStream_t s = static_cast<hipStream_t>(stream);
  void *transposed = static_cast<char *>(workspace) + es * size_t(n) * size_t(n);
  for (int it = 0; it < iterations; ++it) {
    // the product reads a snapshot, so no workgroup sees another's updates; the snapshot's
    // transpose serves the lookup of the first minimising k
    const hipError_t e = dtype == CUASR_AMD_F64 ? snapshot<double>(dist, ld, workspace, n, transposed, n, n, n, s)
                                                : snapshot<float>(dist, ld, workspace, n, transposed, n, n, n, s);
    if (e != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
    FwExtra x;
    x.At = transposed;
    x.ldat = n;
    const int r = fwgemm_run(dtype, n, n, n, workspace, n, workspace, n, dist, ld, parent, ldp, x,
                             CUASR_AMD_KERNEL_AUTO, stream);
    if (r != CUASR_AMD_SUCCESS) return r;
  }
  return CUASR_AMD_SUCCESS;
}

// ---- blocked Floyd-Warshall ------------------------------------------------------------------

extern "C" size_t cuasr_amd_apsp_blocked_workspace_bytes(int dtype, int n) {
  if (n <= 0 || (dtype != CUASR_AMD_F32 && dtype != CUASR_AMD_F64)) return 0;
  const size_t nn = (size_t(n) + 3) & ~size_t(3);
  // block row, block column, transposed block column; then what closing a diagonal block records for its
  // predecessors (fw_close_dist)
  return 3 * size_t(dtype == CUASR_AMD_F64 ? 8 : 4) * FW_BLOCK * (nn + FW_BLOCK);
}

extern "C" int cuasr_amd_apsp_blocked(int dtype, int n, void *dist, int64_t ld, int32_t *parent, int64_t ldp,
                                      void *workspace, void *stream) {
  return cuasr_amd_apsp_blocked_panels(dtype, n, dist, ld, parent, ldp, workspace, CUASR_AMD_PANELS_AUTO, stream);
}

extern "C" int cuasr_amd_apsp_blocked_panels(int dtype, int n, void *dist, int64_t ld, int32_t *parent, int64_t ldp,
                                             void *workspace, int panels, void *stream) {
  if (panels != CUASR_AMD_PANELS_AUTO && panels != CUASR_AMD_PANELS_PAIRED && panels != CUASR_AMD_PANELS_TILED)
    return CUASR_AMD_ERROR_INVALID_PROBLEM;
  const int64_t nn = (int64_t(n) + 3) & ~int64_t(3);
  const int st = check(dtype, n, n, n, workspace, nn > 0 ? nn : 1, workspace, nn > 0 ? nn : 1, dist, ld, parent, ldp,
                       CUASR_AMD_KERNEL_AUTO);
  if (n > 0 && !workspace) return CUASR_AMD_ERROR_WORKSPACE_NULL;
  if (st != CUASR_AMD_SUCCESS) return st;
  if (n == 0) return CUASR_AMD_SUCCESS;
  if (reinterpret_cast<uintptr_t>(workspace) % 16) return CUASR_AMD_ERROR_MISALIGNED_OPERAND;
  const bool f64 = dtype == CUASR_AMD_F64;
  const size_t es = f64 ? 8 : 4;
  hipStream_t s = static_cast<hipStream_t>(stream);
  char *D = static_cast<char *>(dist);
  char *R = static_cast<char *>(workspace);             // block row,    FW_BLOCK x n,  leading dimension FW_BLOCK
  char *C = R + es * FW_BLOCK * size_t(nn);             // block column, n x FW_BLOCK,  leading dimension nn
  char *Ct = C + es * FW_BLOCK * size_t(nn);            // updated block column with k contiguous, leading dimension FW_BLOCK
  char *H = Ct + es * FW_BLOCK * size_t(nn);            // columns, rows and first state of the diagonal block being closed
  // this step's diagonal block had its distances closed during the step before, beside that step's big product;
  // its predecessors are still to be found from what that closure recorded in H
  bool closed = false;
  for (int k0 = 0; k0 < n; k0 += FW_BLOCK) {
    const int bb = n - k0 < FW_BLOCK ? n - k0 : FW_BLOCK;
    char *Dkk = D + es * (size_t(k0) + size_t(k0) * size_t(ld));
    int32_t *Pkk = parent + size_t(k0) + size_t(k0) * size_t(ldp);
    // 1. the diagonal block, closed by one workgroup
    const bool parents_due = closed;
    if (!closed) {
      if (f64)
        launch_kernel(fw_diagonal_kernel<double>, dim3(1), dim3(1024), 0, s, reinterpret_cast<double *>(Dkk), ld, Pkk, ldp, bb, k0);
      else
        launch_kernel(fw_diagonal_kernel<float>, dim3(1), dim3(1024), 0, s, reinterpret_cast<float *>(Dkk), ld, Pkk, ldp, bb, k0);
      if (take_launch_status() != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
    }
    // 2. snapshots of block row and block column (the products below read these, so that no
    //    workgroup sees another's updates)
    char *Drow = D + es * size_t(k0), *Dcol = D + es * size_t(k0) * size_t(ld);
    {
      const int sb0 = ((bb + 63) / 64) * ((n + 63) / 64), sb1 = ((n + 63) / 64) * ((bb + 63) / 64);
      if (f64)
        launch_kernel(snapshot_pair_kernel<double>, dim3(sb0 + sb1), dim3(256), 0, s, reinterpret_cast<const double *>(Drow),
                           reinterpret_cast<double *>(R), int64_t(FW_BLOCK), bb, n, reinterpret_cast<const double *>(Dcol),
                           reinterpret_cast<double *>(C), nn, n, bb, ld, sb0);
      else
        launch_kernel(snapshot_pair_kernel<float>, dim3(sb0 + sb1), dim3(256), 0, s, reinterpret_cast<const float *>(Drow),
                           reinterpret_cast<float *>(R), int64_t(FW_BLOCK), bb, n, reinterpret_cast<const float *>(Dcol),
                           reinterpret_cast<float *>(C), nn, n, bb, ld, sb0);
      if (take_launch_status() != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
    }
    hipError_t e = hipSuccess;
    // 3. block row <- (closed diagonal block) x (block row); block column <- (block column) x (closed
    //    diagonal block).  Neither touches the diagonal block itself (it is closed), so the two are
    //    independent, and while each is too small to fill the chip they share one launch.
    FwExtra x;
    x.k_base = k0;
    int r;
    // below 128 tiles per panel product the two share one launch of the one-thread-per-element kernel;
    // from n = 16257 on each fills the chip on the tiled kernel
    const bool paired = panels == CUASR_AMD_PANELS_AUTO ? (int64_t(n) + 127) / 128 < 128 : panels == CUASR_AMD_PANELS_PAIRED;
    if (paired) {
      const FwArgs g0{bb, n, bb, R + es * size_t(k0) * FW_BLOCK, FW_BLOCK, R, FW_BLOCK, Drow, ld, parent + k0, ldp,
                      nullptr, 0, k0, 0, 0, k0, k0 + bb, nullptr, 0, 0, 0};
      // (the column product also writes the updated column's k-contiguous image for step 4; the rows
      // of the diagonal block, which it skips, are not read there)
      const FwArgs g1{n, bb, bb, C, nn, C + es * size_t(k0), nn, Dcol, ld, parent + size_t(k0) * size_t(ldp), ldp,
                      nullptr, 0, k0, k0, k0 + bb, 0, 0, Ct, FW_BLOCK, 0, 0};
      const int blocks0 = ((bb + 63) / 64) * ((n + 15) / 16), blocks1 = ((n + 63) / 64) * ((bb + 15) / 16);
      const dim3 grid(FW_PARENT_BLOCKS + blocks0 + blocks1);
      if (f64)
        launch_kernel(fwgemm_pair_kernel<double>, grid, dim3(256), 0, s, g0, g1, blocks0,
                      reinterpret_cast<const double *>(parents_due ? H : nullptr), Pkk, ldp, bb, k0);
      else
        launch_kernel(fwgemm_pair_kernel<float>, grid, dim3(256), 0, s, g0, g1, blocks0,
                      reinterpret_cast<const float *>(parents_due ? H : nullptr), Pkk, ldp, bb, k0);
      if (take_launch_status() != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
    } else {
      if (parents_due) {
        if (f64) launch_kernel(fw_parents_kernel<double>, dim3(FW_PARENT_BLOCKS), dim3(256), 0, s, reinterpret_cast<const double *>(H), Pkk, ldp, bb, k0);
        else launch_kernel(fw_parents_kernel<float>, dim3(FW_PARENT_BLOCKS), dim3(256), 0, s, reinterpret_cast<const float *>(H), Pkk, ldp, bb, k0);
        if (take_launch_status() != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
      }
      FwExtra xr = x, xc = x;
      xr.skip_c0 = xc.skip_r0 = k0;
      xr.skip_c1 = xc.skip_r1 = k0 + bb;
      r = fwgemm_run(dtype, bb, n, bb, R + es * size_t(k0) * FW_BLOCK, FW_BLOCK, R, FW_BLOCK, Drow, ld, parent + k0, ldp, xr,
                     CUASR_AMD_KERNEL_VALU, stream);
      if (r != CUASR_AMD_SUCCESS) return r;
      r = fwgemm_run(dtype, n, bb, bb, C, nn, C + es * size_t(k0), nn, Dcol, ld, parent + size_t(k0) * size_t(ldp), ldp, xc,
                     CUASR_AMD_KERNEL_VALU, stream);
      if (r != CUASR_AMD_SUCCESS) return r;
      e = f64 ? snapshot<double>(Dcol, ld, nullptr, 0, Ct, FW_BLOCK, n, bb, s) : snapshot<float>(Dcol, ld, nullptr, 0, Ct, FW_BLOCK, n, bb, s);
      if (e != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
    }
    // 4. everything outside block row and block column <- (block column) x (block row), read in place
    //    (those panels are not written in this step); the column's k-contiguous image serves the lookups.
    //    The next step's diagonal block gets its update first, so that the product's launch can close it
    //    at the same time (fwgemm_tile_kernel).
    closed = false;
    if (k0 + bb < n) {
      x.ahead0 = k0 + bb;
      x.ahead_bb = n - x.ahead0 < FW_BLOCK ? n - x.ahead0 : FW_BLOCK;
      x.hist = H;
      x.closed_ahead = &closed;
    }
    x.At = Ct;
    x.ldat = FW_BLOCK;
    x.skip_r0 = x.skip_c0 = k0;
    x.skip_r1 = x.skip_c1 = k0 + bb;
    if (x.ahead_bb > 0 && !takes_naive_kernel(n, n, CUASR_AMD_KERNEL_AUTO)) {
      // this step's update of that block, by a launch of its own (64 workgroups, a few microseconds): the
      // closure can then start with the big product instead of after one of its tiles
      const int a0 = x.ahead0, abb = x.ahead_bb;
      FwExtra xa;
      xa.k_base = k0;
      r = fwgemm_run(dtype, abb, abb, bb, Dcol + es * size_t(a0), ld, Drow + es * size_t(a0) * size_t(ld), ld,
                     D + es * (size_t(a0) + size_t(a0) * size_t(ld)), ld, parent + size_t(a0) + size_t(a0) * size_t(ldp), ldp,
                     xa, CUASR_AMD_KERNEL_AUTO, stream);
      if (r != CUASR_AMD_SUCCESS) return r;
    } else {
      x.ahead_bb = 0;
    }
    r = fwgemm_run(dtype, n, n, bb, Dcol, ld, Drow, ld, dist, ld, parent, ldp, x, CUASR_AMD_KERNEL_AUTO, stream);
    if (r != CUASR_AMD_SUCCESS) return r;
  }
  return CUASR_AMD_SUCCESS;
}
