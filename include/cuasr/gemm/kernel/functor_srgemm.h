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

template <typename T> struct Tile {
  static constexpr int VW = 16 / sizeof(T);
  static constexpr int TM = 8, TN = sizeof(T) == 8 ? 4 : 8;
  static constexpr int BM = 16 * TM, BN = 16 * TN, BK = 16;
  static constexpr int HM = TM / VW, GN = TN / VW;
  static constexpr int LDA = BM + VW, LDB = BN + VW;
  static constexpr int A_VECS = BM * BK / VW / 256, B_VECS = BN * BK / VW / 256;
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "4- and 8-byte element types");
  typedef T vec_t __attribute__((ext_vector_type(VW)));
  // the same vector in global memory, where only element alignment is required
  typedef T gvec_t __attribute__((ext_vector_type(VW), aligned(sizeof(T))));
};

// how an operand's panel is fetched: along which direction its 16-byte vectors run
enum PanelMode { kElements = 0, kVectorsAlongX = 1, kVectorsAlongK = 2 };

// Global -> registers: VECS vectors per thread of a ROWS x BK panel whose first row / column is x0 and first k
// is k0.  Indices outside [0, x_end) x [0, k_end) are clamped to the last valid one: what is fetched there is
// never used (rows and columns past the edge are not stored, k past the end is not iterated).
template <typename T, int ROWS, int VECS>
__device__ __forceinline__ void load_panel(typename Tile<T>::vec_t (&r)[VECS], const T *base, long long s_x, long long s_k,
                                           int x0, int x_end, int k0, int k_end, int mode) {
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

// (two waves per SIMD at least: without the attribute the compiler may take all 512 registers of a lane)
template <typename AddOp, typename MultOp, typename T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void functor_srgemm_kernel(FunctorSrgemmParams<T> p) {
  using namespace functor_detail;
  using Ti = Tile<T>;
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

  // one k of the panels in LDS: the thread's 8 rows of A and 8 (4) columns of B
  struct Fragment {
    vec_t a[HM], b[GN];
  };
  auto fetch = [&](Fragment &f, int cur, int kk) {
#pragma unroll
    for (int g = 0; g < HM; ++g) f.a[g] = *reinterpret_cast<const vec_t *>(&As[cur][kk][g * 16 * VW + ty * VW]);
#pragma unroll
    for (int g = 0; g < GN; ++g) f.b[g] = *reinterpret_cast<const vec_t *>(&Bs[cur][kk][g * 16 * VW + tx * VW]);
  };
  auto compute = [&](const Fragment &f) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = add_op(opaque(mult_op(f.a[i / VW][i % VW], f.b[j / VW][j % VW])), acc[i][j]);
  };

  if (ke > kb) {
    vec_t ra[Ti::A_VECS], rb[Ti::B_VECS];
    load_panel<T, BM, Ti::A_VECS>(ra, p.A, p.sa_m, p.sa_k, m0, p.m, kb, ke, a_mode);
    load_panel<T, BN, Ti::B_VECS>(rb, p.B, p.sb_n, p.sb_k, n0, p.n, kb, ke, b_mode);
    store_panel<T, BM, Ti::LDA, Ti::A_VECS>(As[0], ra, a_mode);
    store_panel<T, BN, Ti::LDB, Ti::B_VECS>(Bs[0], rb, b_mode);
    __syncthreads();
    int cur = 0;
    for (int k0 = kb; k0 < ke; k0 += BK) {
      const bool more = k0 + BK < ke;
      if (more) {
        load_panel<T, BM, Ti::A_VECS>(ra, p.A, p.sa_m, p.sa_k, m0, p.m, k0 + BK, ke, a_mode);
        load_panel<T, BN, Ti::B_VECS>(rb, p.B, p.sb_n, p.sb_k, n0, p.n, k0 + BK, ke, b_mode);
      }
      if (k0 + BK <= ke) {
        // whole k-tile, two k at a time: the reads of the next pair are issued before the current pair is
        // computed (two fragment sets), and nothing moves across a pair's boundary -- left alone, the
        // scheduler hoists the whole tile's reads and the kernel ends up with one wave per SIMD
        Fragment f[2][2];
        fetch(f[0][0], cur, 0);
        fetch(f[0][1], cur, 1);
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
          const int s = (kk >> 1) & 1;
          if (kk + 2 < BK) {
            fetch(f[s ^ 1][0], cur, kk + 2);
            fetch(f[s ^ 1][1], cur, kk + 3);
          }
          compute(f[s][0]);
          compute(f[s][1]);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        for (int kk = 0; kk < ke - k0; ++kk) {
          Fragment f;
          fetch(f, cur, kk);
          compute(f);
        }
      }
      if (more) {
        store_panel<T, BM, Ti::LDA, Ti::A_VECS>(As[cur ^ 1], ra, a_mode);
        store_panel<T, BN, Ti::LDB, Ti::B_VECS>(Bs[cur ^ 1], rb, b_mode);
      }
      __syncthreads();
      cur ^= 1;
    }
  }

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
/// side (grid dimension y) and no epilogue is applied.
template <typename AddOp, typename MultOp, typename T>
inline hipError_t launch_functor_srgemm(FunctorSrgemmParams<T> const &p, hipStream_t stream) {
  using Ti = functor_detail::Tile<T>;
  if (p.m <= 0 || p.n <= 0) return hipSuccess;
  const long long tiles = (long long)((p.m + Ti::BM - 1) / Ti::BM) * ((p.n + Ti::BN - 1) / Ti::BN);
  const int slices = p.workspace ? p.slices : 1;
  if (tiles > 0x7fffffffLL || slices < 1 || slices > 65535) return hipErrorInvalidValue;
  void *args[] = {const_cast<void *>(static_cast<const void *>(&p))};
  return hipLaunchKernel(reinterpret_cast<const void *>(&functor_srgemm_kernel<AddOp, MultOp, T>),
                         dim3((unsigned)tiles, (unsigned)slices), dim3(256), args, 0, stream);
}

}  // namespace kernel
}  // namespace gemm
}  // namespace cuasr
