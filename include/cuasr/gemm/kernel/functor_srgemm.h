// SRGEMM instantiated from arbitrary user functors -- the reference builds every kernel from whatever
// operator() the user writes (include/cuasr/arch/srmma.h:65-92 of the reference,
// examples/01_userdefined_semiring/userdefined_semiring.cu:56-99).  The library's tuned kernels cover the
// operators of cuasr/functional.h; a functor type that names none of them (no cuasr::op_tag
// specialisation) is compiled into this kernel instead, in the user's own translation unit, which
// therefore has to be compiled by hipcc.  The functors need a __host__ __device__ operator()(T, T); the
// addition functor the static member Identity, the multiplication functor Identity and Annihilator, as in
// the reference.
//
// Results are those of the reference's host SRGEMM
// (tools/include/cuasr/reference/srgemm/host_srgemm.h:33-113) for ANY functor pair, associative or not:
// every output element is accumulated by one thread, accum = add(mult(a, b), accum) for k ascending from
// AddOp::Identity, then D = add(mult(alpha, accum), mult(beta, C)), or mult(alpha, accum) when the source
// is not needed (epilogue/thread/semiring_linear_combination.h:118-125, :152-183).  Whether a floating-point
// product is fused with the add that consumes it -- inside a functor's own body, or a mult's product into the
// add functor's sum -- follows the translation unit's -ffp-contract setting: hipcc by default fuses a * b + c
// on the device and not on the host (as nvcc does for the reference's kernels), so compile with
//     hipcc -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops
// where the device has to match the host reference bit for bit (the second flag keeps packed-fp32 instructions
// out of the kernel, as in every object of the library).
//
// The tile (gfx950, 64-wide waves):
//   * workgroup 256 threads = 4 waves as 16 x 16 threads; output tile 128 x 128 for 4-byte elements (a thread
//     owns 8 x 8 accumulators), 128 x 64 for 8-byte elements (8 x 4); k-tile 16.  A thread's rows and columns
//     come in groups of one 16-byte vector (4 or 2 elements), the groups 16 vectors apart, so that every LDS
//     fragment read is one 16-byte read, conflict-free (16 lanes read 256 consecutive bytes of the B panel, the
//     A panel's address is shared by those 16 lanes).
//   * A and B panels k-major in LDS ([k][row], [k][column]), double buffered, ONE barrier per k-tile: the
//     next tile's global loads are issued before the current tile is computed and stored to the other
//     buffer after it.
//   * global loads are 16-byte vectors along whichever direction of the operand is contiguous (rows: stored
//     to LDS as they are; k: transposed on the way, consecutive lanes to consecutive banks); only element
//     alignment is assumed (the hardware takes 16-byte accesses at any element boundary); a vector that
//     would cross the matrix edge or the end of the k range is fetched element by element, clamped.
//   * a ragged last k-tile shortens the loop -- never pads: a padded identity is not neutral for every
//     functor pair (the reference pads, threadblock/srmma_pipelined.h:172-173, which is only right for pairs
//     whose mult(identity, x) is absorbing).
//   * blockIdx.x walks the output tiles so that the workgroups resident on one XCD (blockIdx.x mod 8) cover
//     a compact 8-row block of tiles and share A and B panels in that XCD's L2; blockIdx.y is the split-K
//     slice.
//   * split-K (workspace != null): slice z accumulates its k range from AddOp::Identity and stores the raw
//     accumulators to workspace[z][m][n] (row-major); the reduction kernels of
//     cuasr/reduction/kernel/reduce_split_k.h finish the job.
#pragma once
#include <hip/hip_runtime.h>

#include <type_traits>

namespace cuasr {
namespace gemm {
namespace kernel {

template <typename T> struct FunctorSrgemmParams {
  int m, n, k;
  const T *A; long long sa_m, sa_k;   // A[i][kk] at A + i * sa_m + kk * sa_k
  const T *B; long long sb_k, sb_n;
  const T *C; long long sc_m, sc_n;
  T *D;       long long sd_m, sd_n;
  T alpha, beta;
  const T *alpha_ptr, *beta_ptr;      // device pointers that override alpha / beta when not null
  // split-K: slice z covers k in [min(k, z * k_per_slice), min(k, (z + 1) * k_per_slice)), and the last slice
  // runs on to k when last_takes_rest is set (the parallel form's rule)
  T *workspace;                        // null: one slice, epilogue in the kernel
  int slices, k_per_slice, last_takes_rest;
};

namespace functor_detail {

// With CUASR_AMD_FUNCTOR_FENCE defined to 1, a floating-point product passes through an empty asm statement on
// its way into the add, so that the two are never fused whatever -ffp-contract says (integer multiply-adds are
// exact: nothing to keep apart).  Off by default: the fence only separates mult from add -- what happens inside
// a functor's own body follows -ffp-contract anyway, so that flag is what a bit-exact build needs -- and it
// hides from the compiler that the product is a canonical number, which costs functors built on fminf / fmaxf
// one more instruction per term.
#ifndef CUASR_AMD_FUNCTOR_FENCE
#define CUASR_AMD_FUNCTOR_FENCE 0
#endif
template <typename T> __device__ __forceinline__ T opaque(T v) {
#if CUASR_AMD_FUNCTOR_FENCE
  if constexpr (std::is_floating_point<T>::value) asm("" : "+v"(v));
#endif
  return v;
}

// SMALL: a quarter of the tile (4 x 4 accumulators per thread for 4-byte elements, 4 x 2 for 8-byte ones) for
// outputs whose full-size tiles would leave most of the chip without work
template <typename T, bool SMALL = false> struct Tile {
  static constexpr int VW = 16 / sizeof(T);
  static constexpr int TM = SMALL ? 4 : 8, TN = (SMALL ? 4 : 8) / (sizeof(T) == 8 ? 2 : 1);
#ifndef CUASR_AMD_FUNCTOR_BK
#define CUASR_AMD_FUNCTOR_BK 16
#endif
  static constexpr int BM = 16 * TM, BN = 16 * TN, BK = CUASR_AMD_FUNCTOR_BK;
  static constexpr int HM = TM / VW, GN = TN / VW;
  static constexpr int LDA = BM + VW, LDB = BN + VW;
  static_assert(BM * BK / VW >= 256 && BN * BK / VW >= 256, "a panel gives every thread a vector");
  static constexpr int A_VECS = BM * BK / VW / 256, B_VECS = BN * BK / VW / 256;
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "4- and 8-byte element types");
  typedef T vec_t __attribute__((ext_vector_type(VW)));
  // the same vector in global memory, where only element alignment is required
  typedef T gvec_t __attribute__((ext_vector_type(VW), aligned(sizeof(T))));
};

// how an operand's panel is fetched: along which direction its 16-byte vectors run
enum PanelMode { kElements = 0, kVectorsAlongX = 1, kVectorsAlongK = 2 };

// Global -> registers, the guarded form: VECS vectors per thread of a ROWS x BK panel whose first row / column
// is x0 and first k is k0, for any strides and any position.  Indices outside [0, x_end) x [0, k_end) are
// clamped to the last valid one: what is fetched there is never used (rows and columns past the edge are not
// stored, k past the end is not iterated).  A vector that lies wholly inside is one 16-byte load.
template <typename T, int ROWS, int VECS>
__device__ __forceinline__ void load_panel_guarded(typename Tile<T>::vec_t (&r)[VECS], const T *base, long long s_x,
                                                   long long s_k, int x0, int x_end, int k0, int k_end, int mode) {
  using Ti = Tile<T>;
  constexpr int VW = Ti::VW;
  const int tid = threadIdx.x;
  if (mode == kVectorsAlongK) {
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      const int v = tid + 256 * p;
      const long long gx = min(x0 + v % ROWS, x_end - 1);
      const int gk = k0 + (v / ROWS) * VW;
      const T *src = base + gx * s_x;
      if (gk + VW <= k_end) {
        r[p] = *reinterpret_cast<const typename Ti::gvec_t *>(src + gk);
      } else {
#pragma unroll
        for (int e = 0; e < VW; ++e) r[p][e] = src[min(gk + e, k_end - 1)];
      }
    }
  } else {
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      const int v = tid + 256 * p;
      const int gx = x0 + (v % (ROWS / VW)) * VW;
      const long long gk = min(k0 + v / (ROWS / VW), k_end - 1);
      const T *src = base + gk * s_k;
      if (mode == kVectorsAlongX && gx + VW <= x_end) {
        r[p] = *reinterpret_cast<const typename Ti::gvec_t *>(src + gx);
      } else {
#pragma unroll
        for (int e = 0; e < VW; ++e) r[p][e] = src[(long long)min(gx + e, x_end - 1) * s_x];
      }
    }
  }
}

// Global -> registers, the fast form, for a panel that lies wholly inside the matrix and the k range: a thread's
// vectors sit at fixed 32-bit byte offsets from the panel's first element, whose address is the same for the
// whole workgroup (a scalar register pair that moves on by one k-tile per iteration) -- one register per vector
// instead of an address pair and its guards.
template <typename T, int ROWS, int VECS, int MODE> struct FastPanel {
  using Ti = Tile<T>;
  unsigned offset[VECS];
  __device__ __forceinline__ void init(long long s_x, long long s_k) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      const int v = tid + 256 * p;
      if (MODE == kVectorsAlongK) offset[p] = (unsigned)(((long long)(v % ROWS) * s_x + (v / ROWS) * Ti::VW) * (long long)sizeof(T));
      else offset[p] = (unsigned)(((long long)(v / (ROWS / Ti::VW)) * s_k + (v % (ROWS / Ti::VW)) * Ti::VW) * (long long)sizeof(T));
    }
  }
  __device__ __forceinline__ void load(typename Ti::vec_t (&r)[VECS], const T *panel) const {
#pragma unroll
    for (int p = 0; p < VECS; ++p)
      r[p] = *reinterpret_cast<const typename Ti::gvec_t *>(reinterpret_cast<const char *>(panel) + offset[p]);
  }
  // do all of a panel's offsets fit 32 bits?
  static __device__ __forceinline__ bool fits(long long s_x, long long s_k) {
    const long long last = MODE == kVectorsAlongK ? (long long)(ROWS - 1) * s_x + Ti::BK : (long long)(Ti::BK - 1) * s_k + ROWS;
    return last * (long long)sizeof(T) < (1LL << 32);
  }
};

// registers -> LDS, k-major.  A vector along x is stored as it is; a vector along k is transposed, the lanes of
// a store instruction going to consecutive x, i.e. consecutive banks.
template <typename T, int ROWS, int LD, int VECS>
__device__ __forceinline__ void store_panel(T (*panel)[LD], const typename Tile<T>::vec_t (&r)[VECS], int mode) {
  using Ti = Tile<T>;
  constexpr int VW = Ti::VW;
  const int tid = threadIdx.x;
  if (mode == kVectorsAlongK) {
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      const int v = tid + 256 * p;
      const int xx = v % ROWS, kk = (v / ROWS) * VW;
#pragma unroll
      for (int e = 0; e < VW; ++e) panel[kk + e][xx] = r[p][e];
    }
  } else {
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      const int v = tid + 256 * p;
      const int xx = (v % (ROWS / VW)) * VW, kk = v / (ROWS / VW);
      *reinterpret_cast<typename Ti::vec_t *>(&panel[kk][xx]) = r[p];
    }
  }
}

// Output tile of workgroup `bid`: tiles are walked in blocks of 8 tile rows, column by column inside a block,
// and the walk is cut into 8 equal runs, one per XCD (workgroup ids are dealt to the 8 XCDs in turn), so that
// the workgroups an XCD holds at one time sit in one compact block and share its panels in that XCD's L2.
__device__ __forceinline__ void tile_coords(int bid, int tiles_m, int tiles_n, int &tm, int &tn) {
  const int tiles = tiles_m * tiles_n;
  int t = bid;
  if (tiles % 8 == 0) t = (bid % 8) * (tiles / 8) + bid / 8;
  constexpr int GM = 8;
  const int group = t / (GM * tiles_n), first = group * GM;
  const int rows = min(tiles_m - first, GM), r = t - group * GM * tiles_n;
  tm = first + r % rows;
  tn = r / rows;
}

}  // namespace functor_detail

// (CUASR_AMD_FUNCTOR_WAVES waves per SIMD at least: without the attribute the compiler may take all 512 registers of a lane)
#ifndef CUASR_AMD_FUNCTOR_WAVES
#define CUASR_AMD_FUNCTOR_WAVES 2
#endif

/// The kernel's pieces, as static members so that the main loop can be instantiated per pair of panel forms.
template <typename AddOp, typename MultOp, typename T, bool SMALL> struct FunctorSrgemmBody {
  using Ti = functor_detail::Tile<T, SMALL>;
  using vec_t = typename Ti::vec_t;
  static constexpr int VW = Ti::VW, TM = Ti::TM, TN = Ti::TN, BM = Ti::BM, BN = Ti::BN, BK = Ti::BK, HM = Ti::HM, GN = Ti::GN;
  typedef T APanel[BK][Ti::LDA];
  typedef T BPanel[BK][Ti::LDB];

  // one k of the panels in LDS: the thread's 8 rows of A and 8 (4) columns of B
  struct Fragment {
    vec_t a[HM], b[GN];
  };
  static __device__ __forceinline__ void fetch(Fragment &f, const APanel &as, const BPanel &bs, int kk, int ty, int tx) {
#pragma unroll
    for (int g = 0; g < HM; ++g) f.a[g] = *reinterpret_cast<const vec_t *>(&as[kk][g * 16 * VW + ty * VW]);
#pragma unroll
    for (int g = 0; g < GN; ++g) f.b[g] = *reinterpret_cast<const vec_t *>(&bs[kk][g * 16 * VW + tx * VW]);
  }
  static __device__ __forceinline__ void terms(T (&acc)[TM][TN], const Fragment &f) {
    AddOp add_op;
    MultOp mult_op;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = add_op(functor_detail::opaque(mult_op(f.a[i / VW][i % VW], f.b[j / VW][j % VW])), acc[i][j]);
  }
  // a whole k-tile, two k at a time: the reads of the next pair are issued before the current pair is computed
  // (two fragment sets), and nothing moves across a pair's boundary -- left alone, the scheduler hoists the
  // whole tile's reads and the kernel ends up with one wave per SIMD
  static __device__ __forceinline__ void whole_tile(T (&acc)[TM][TN], const APanel &as, const BPanel &bs, int ty, int tx) {
    Fragment f[2][2];
    fetch(f[0][0], as, bs, 0, ty, tx);
    fetch(f[0][1], as, bs, 1, ty, tx);
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      const int s = (kk >> 1) & 1;
      if (kk + 2 < BK) {
        fetch(f[s ^ 1][0], as, bs, kk + 2, ty, tx);
        fetch(f[s ^ 1][1], as, bs, kk + 3, ty, tx);
      }
      terms(acc, f[s][0]);
      terms(acc, f[s][1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  static __device__ __forceinline__ void part_tile(T (&acc)[TM][TN], const APanel &as, const BPanel &bs, int kcount, int ty, int tx) {
    for (int kk = 0; kk < kcount; ++kk) {
      Fragment f;
      fetch(f, as, bs, kk, ty, tx);
      terms(acc, f);
    }
  }

  // `tiles` whole k-tiles of panels that lie wholly inside the matrix, fetched in their fast form.  Branch-free
  // inside: every iteration fetches the next tile (the last one fetches itself again), computes, stores, and
  // passes one barrier; the loads of tile t + 1 are in flight while tile t is computed.
  template <int A_MODE, int B_MODE>
  static __device__ __forceinline__ void fast_tiles(T (&acc)[TM][TN], APanel *As, BPanel *Bs, const T *a_panel, long long sa_x, long long sa_k,
                                                    const T *b_panel, long long sb_x, long long sb_k, int tiles, int ty, int tx) {
    using namespace functor_detail;
    FastPanel<T, BM, Ti::A_VECS, A_MODE> fa;
    FastPanel<T, BN, Ti::B_VECS, B_MODE> fb;
    fa.init(sa_x, sa_k);
    fb.init(sb_x, sb_k);
    const long long a_step = (long long)BK * sa_k, b_step = (long long)BK * sb_k;
    vec_t ra[Ti::A_VECS], rb[Ti::B_VECS];
    fa.load(ra, a_panel);
    fb.load(rb, b_panel);
    store_panel<T, BM, Ti::LDA, Ti::A_VECS>(As[0], ra, A_MODE);
    store_panel<T, BN, Ti::LDB, Ti::B_VECS>(Bs[0], rb, B_MODE);
    __syncthreads();
    for (int t = 0; t < tiles; ++t) {
      const int next = min(t + 1, tiles - 1), cur = t & 1;
      fa.load(ra, a_panel + next * a_step);
      fb.load(rb, b_panel + next * b_step);
      whole_tile(acc, As[cur], Bs[cur], ty, tx);
      store_panel<T, BM, Ti::LDA, Ti::A_VECS>(As[cur ^ 1], ra, A_MODE);
      store_panel<T, BN, Ti::LDB, Ti::B_VECS>(Bs[cur ^ 1], rb, B_MODE);
      __syncthreads();
    }
  }

  // k in [kb, ke) with every guard: any strides, panels that reach past the matrix edge, a ragged last k-tile
  static __device__ __forceinline__ void guarded_tiles(T (&acc)[TM][TN], APanel *As, BPanel *Bs, FunctorSrgemmParams<T> const &p, int m0, int n0,
                                                       int kb, int ke, int a_mode, int b_mode, int ty, int tx) {
    using namespace functor_detail;
    vec_t ra[Ti::A_VECS], rb[Ti::B_VECS];
    load_panel_guarded<T, BM, Ti::A_VECS>(ra, p.A, p.sa_m, p.sa_k, m0, p.m, kb, ke, a_mode);
    load_panel_guarded<T, BN, Ti::B_VECS>(rb, p.B, p.sb_n, p.sb_k, n0, p.n, kb, ke, b_mode);
    store_panel<T, BM, Ti::LDA, Ti::A_VECS>(As[0], ra, a_mode);
    store_panel<T, BN, Ti::LDB, Ti::B_VECS>(Bs[0], rb, b_mode);
    __syncthreads();
    int cur = 0;
    for (int k0 = kb; k0 < ke; k0 += BK) {
      const bool more = k0 + BK < ke;
      if (more) {
        load_panel_guarded<T, BM, Ti::A_VECS>(ra, p.A, p.sa_m, p.sa_k, m0, p.m, k0 + BK, ke, a_mode);
        load_panel_guarded<T, BN, Ti::B_VECS>(rb, p.B, p.sb_n, p.sb_k, n0, p.n, k0 + BK, ke, b_mode);
      }
      if (k0 + BK <= ke) whole_tile(acc, As[cur], Bs[cur], ty, tx);
      else part_tile(acc, As[cur], Bs[cur], ke - k0, ty, tx);
      if (more) {
        store_panel<T, BM, Ti::LDA, Ti::A_VECS>(As[cur ^ 1], ra, a_mode);
        store_panel<T, BN, Ti::LDB, Ti::B_VECS>(Bs[cur ^ 1], rb, b_mode);
      }
      __syncthreads();
      cur ^= 1;
    }
  }
};

template <typename AddOp, typename MultOp, typename T, bool SMALL = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(CUASR_AMD_FUNCTOR_WAVES))) void functor_srgemm_kernel(FunctorSrgemmParams<T> p) {
  using namespace functor_detail;
  using Body = FunctorSrgemmBody<AddOp, MultOp, T, SMALL>;
  using Ti = Tile<T, SMALL>;
  using vec_t = typename Ti::vec_t;
  using gvec_t = typename Ti::gvec_t;
  constexpr int VW = Ti::VW, TM = Ti::TM, TN = Ti::TN, BM = Ti::BM, BN = Ti::BN, BK = Ti::BK, HM = Ti::HM, GN = Ti::GN;
  __shared__ __attribute__((aligned(16))) T As[2][BK][Ti::LDA];
  __shared__ __attribute__((aligned(16))) T Bs[2][BK][Ti::LDB];
  AddOp add_op;
  MultOp mult_op;
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  int tm, tn;
  tile_coords((int)blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // this workgroup's k range
  int kb = 0, ke = p.k;
  if (p.workspace) {
    const int z = (int)blockIdx.y;
    const long long b = (long long)z * p.k_per_slice, e = b + p.k_per_slice;
    kb = (int)(b < p.k ? b : p.k);
    ke = (z + 1 == p.slices && p.last_takes_rest) ? p.k : (int)(e < p.k ? e : p.k);
    if (ke < kb) ke = kb;
  }

  T acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = AddOp::Identity;

  const int a_mode = p.sa_m == 1 ? kVectorsAlongX : p.sa_k == 1 ? kVectorsAlongK : kElements;
  const int b_mode = p.sb_n == 1 ? kVectorsAlongX : p.sb_k == 1 ? kVectorsAlongK : kElements;

  // the whole k-tiles of a tile that lies wholly inside the output run in the branch-free loop of their pair of
  // panel forms; everything else -- tiles on the edge, strides that are not 1 in either direction, operands so
  // large that a panel's byte offsets outgrow 32 bits, and the ragged last k-tile -- in the guarded loop
  int k_done = kb;
  const int whole = (ke - kb) / BK;
  if (whole > 0 && m0 + BM <= p.m && n0 + BN <= p.n && a_mode != kElements && b_mode != kElements) {
    const T *a_panel = p.A + (long long)m0 * p.sa_m + (long long)kb * p.sa_k;
    const T *b_panel = p.B + (long long)n0 * p.sb_n + (long long)kb * p.sb_k;
    bool done = true;
    if (a_mode == kVectorsAlongX && b_mode == kVectorsAlongX && FastPanel<T, BM, Ti::A_VECS, kVectorsAlongX>::fits(p.sa_m, p.sa_k) &&
        FastPanel<T, BN, Ti::B_VECS, kVectorsAlongX>::fits(p.sb_n, p.sb_k))
      Body::template fast_tiles<kVectorsAlongX, kVectorsAlongX>(acc, As, Bs, a_panel, p.sa_m, p.sa_k, b_panel, p.sb_n, p.sb_k, whole, ty, tx);
    else if (a_mode == kVectorsAlongX && b_mode == kVectorsAlongK && FastPanel<T, BM, Ti::A_VECS, kVectorsAlongX>::fits(p.sa_m, p.sa_k) &&
             FastPanel<T, BN, Ti::B_VECS, kVectorsAlongK>::fits(p.sb_n, p.sb_k))
      Body::template fast_tiles<kVectorsAlongX, kVectorsAlongK>(acc, As, Bs, a_panel, p.sa_m, p.sa_k, b_panel, p.sb_n, p.sb_k, whole, ty, tx);
    else if (a_mode == kVectorsAlongK && b_mode == kVectorsAlongX && FastPanel<T, BM, Ti::A_VECS, kVectorsAlongK>::fits(p.sa_m, p.sa_k) &&
             FastPanel<T, BN, Ti::B_VECS, kVectorsAlongX>::fits(p.sb_n, p.sb_k))
      Body::template fast_tiles<kVectorsAlongK, kVectorsAlongX>(acc, As, Bs, a_panel, p.sa_m, p.sa_k, b_panel, p.sb_n, p.sb_k, whole, ty, tx);
    else if (a_mode == kVectorsAlongK && b_mode == kVectorsAlongK && FastPanel<T, BM, Ti::A_VECS, kVectorsAlongK>::fits(p.sa_m, p.sa_k) &&
             FastPanel<T, BN, Ti::B_VECS, kVectorsAlongK>::fits(p.sb_n, p.sb_k))
      Body::template fast_tiles<kVectorsAlongK, kVectorsAlongK>(acc, As, Bs, a_panel, p.sa_m, p.sa_k, b_panel, p.sb_n, p.sb_k, whole, ty, tx);
    else
      done = false;
    if (done) k_done = kb + whole * BK;
  }
  if (k_done < ke) Body::guarded_tiles(acc, As, Bs, p, m0, n0, k_done, ke, a_mode, b_mode, ty, tx);

  auto row_of = [&](int i) { return m0 + (i / VW) * 16 * VW + ty * VW + i % VW; };
  auto col_of = [&](int j) { return n0 + (j / VW) * 16 * VW + tx * VW + j % VW; };

  if (p.workspace) {
    // raw accumulators of this slice, row-major m x n
    T *ws = p.workspace + (long long)blockIdx.y * p.m * p.n;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = row_of(i);
      if (row >= p.m) continue;
#pragma unroll
      for (int g = 0; g < GN; ++g) {
        const int col = col_of(g * VW);
        T *dst = ws + (long long)row * p.n + col;
        if (col + VW <= p.n) {
          vec_t o;
#pragma unroll
          for (int e = 0; e < VW; ++e) o[e] = acc[i][g * VW + e];
          *reinterpret_cast<gvec_t *>(dst) = o;
        } else {
#pragma unroll
          for (int e = 0; e < VW; ++e)
            if (col + e < p.n) dst[e] = acc[i][g * VW + e];
        }
      }
    }
    return;
  }

  const T alpha = p.alpha_ptr ? *p.alpha_ptr : p.alpha, beta = p.beta_ptr ? *p.beta_ptr : p.beta;
  const bool source_needed = !(AddOp::Identity == mult_op(beta, MultOp::Identity));
  auto finish = [&](T a, T c) {
    const T scaled = opaque(mult_op(alpha, a));
    return source_needed ? add_op(scaled, opaque(mult_op(beta, c))) : scaled;
  };
  if (p.sd_n == 1 && (!source_needed || p.sc_n == 1)) {
    // rows of D are contiguous: 16-byte accesses along a row
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = row_of(i);
      if (row >= p.m) continue;
#pragma unroll
      for (int g = 0; g < GN; ++g) {
        const int col = col_of(g * VW);
        T *dst = p.D + (long long)row * p.sd_m + col;
        const T *src = p.C + (long long)row * p.sc_m + col;
        if (col + VW <= p.n) {
          vec_t c{}, o;
          if (source_needed) c = *reinterpret_cast<const gvec_t *>(src);
#pragma unroll
          for (int e = 0; e < VW; ++e) o[e] = finish(acc[i][g * VW + e], c[e]);
          *reinterpret_cast<gvec_t *>(dst) = o;
        } else {
#pragma unroll
          for (int e = 0; e < VW; ++e)
            if (col + e < p.n) dst[e] = finish(acc[i][g * VW + e], source_needed ? src[e] : T());
        }
      }
    }
  } else if (p.sd_m == 1 && (!source_needed || p.sc_m == 1)) {
    // columns of D are contiguous: 16-byte accesses along a column
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = col_of(j);
      if (col >= p.n) continue;
#pragma unroll
      for (int g = 0; g < HM; ++g) {
        const int row = row_of(g * VW);
        T *dst = p.D + (long long)col * p.sd_n + row;
        const T *src = p.C + (long long)col * p.sc_n + row;
        if (row + VW <= p.m) {
          vec_t c{}, o;
          if (source_needed) c = *reinterpret_cast<const gvec_t *>(src);
#pragma unroll
          for (int e = 0; e < VW; ++e) o[e] = finish(acc[g * VW + e][j], c[e]);
          *reinterpret_cast<gvec_t *>(dst) = o;
        } else {
#pragma unroll
          for (int e = 0; e < VW; ++e)
            if (row + e < p.m) dst[e] = finish(acc[g * VW + e][j], source_needed ? src[e] : T());
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = row_of(i);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int col = col_of(j);
        if (row < p.m && col < p.n)
          p.D[row * p.sd_m + col * p.sd_n] = finish(acc[i][j], source_needed ? p.C[row * p.sc_m + col * p.sc_n] : T());
      }
    }
  }
}

/// Launch on `stream`; hipSuccess or the launch's error.  With p.workspace set, p.slices slices run side by
/// side (grid dimension y) and no epilogue is applied.  The quarter-size tile is launched when the full-size
/// one would give the chip's 256 compute units fewer than two workgroups each.
template <typename AddOp, typename MultOp, typename T>
inline hipError_t launch_functor_srgemm(FunctorSrgemmParams<T> const &p, hipStream_t stream) {
  using Full = functor_detail::Tile<T, false>;
  using Quarter = functor_detail::Tile<T, true>;
  if (p.m <= 0 || p.n <= 0) return hipSuccess;
  const int slices = p.workspace ? p.slices : 1;
  if (slices < 1 || slices > 65535) return hipErrorInvalidValue;
  long long tiles = (long long)((p.m + Full::BM - 1) / Full::BM) * ((p.n + Full::BN - 1) / Full::BN);
  const bool quarter = tiles * slices < 512;
  if (quarter) tiles = (long long)((p.m + Quarter::BM - 1) / Quarter::BM) * ((p.n + Quarter::BN - 1) / Quarter::BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  void *args[] = {const_cast<void *>(static_cast<const void *>(&p))};
  const void *fn = quarter ? reinterpret_cast<const void *>(&functor_srgemm_kernel<AddOp, MultOp, T, true>)
                           : reinterpret_cast<const void *>(&functor_srgemm_kernel<AddOp, MultOp, T, false>);
  return hipLaunchKernel(fn, dim3((unsigned)tiles, (unsigned)slices), dim3(256), args, 0, stream);
}

}  // namespace kernel
}  // namespace gemm
}  // namespace cuasr
