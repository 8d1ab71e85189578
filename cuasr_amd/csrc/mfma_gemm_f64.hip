// plus-times ("control") semiring for double on the matrix cores:
//     D = alpha * (A . B) + beta * C      with v_mfma_f64_16x16x4_f64
//
// Replaces, for this pair and type, the reference's SIMT kernel
// (include/cuasr/gemm/kernel/srgemm.h:156-321 with
// DefaultSemiRingConfiguration<plus<double>, multiplies<double>>,
// include/cuasr/gemm/device/default_srgemm_configuration.h:44-72).  The sum
// over k is formed in the instruction's order (groups of 4 k, fused
// multiply-adds), not the host reference's sequential unfused order: results
// agree with it to rounding -- |d - r| <= 1e-12 * sum_k |a||b| -- not bit for
// bit; the vector-ALU tile (kernel = VALU) stays available for a bit-exact one.
//
// Workgroup 256 threads = 4 waves (2 x 2), output tile 128 x 128, wave tile
// 64 x 64 = 4 x 4 blocks of 16 x 16 (64 accumulator doubles per lane), k-tile
// 16.  The instruction takes, per lane l, A[row l % 16][k = l / 16] and
// B[k = l / 16][column l % 16]; the block's result has row l / 16 + 4 * r,
// column l % 16 in register r = 0..3 of lane l.  LDS panels are k-major,
// [k][LD] doubles: a fragment read is 16 consecutive doubles of 4 consecutive
// rows, one ds_read_b64 per lane.
#include "semiring.h"

namespace cuasr_amd {

bool mfma_direct_f64_can_run(const Problem &);                // mfma_direct_f64.hip
hipError_t mfma_direct_f64_launch(const Problem &, hipStream_t);

namespace gemm_mfma_f64 {

typedef double v2d __attribute__((ext_vector_type(2)));
typedef double v4d __attribute__((ext_vector_type(4)));

constexpr int BM = 128, BN = 128, BK = 16, LD = 128 + 8, VECS = BM * BK / 2 / 256;  // 4 vectors per thread and panel

struct Smem {
  double a[2][BK][LD];
  double b[2][BK][LD];
};

__device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int &bm, int &bn) {
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

// One operand's share of a thread in the global -> LDS copy of a 128 x 16 panel:
// four 16-byte vectors (x contiguous: 2 consecutive x at one k; k contiguous: 2
// consecutive k at one x).  src[] points at the vectors of the first k-tile, x
// clamped to the matrix, and advances by one k-tile per load.
// LOOSE: operands of any extent, leading dimension and 8-byte alignment.  The vector loads are made at element
// alignment, and a vector that would cross the end of its row (x contiguous) or of the k range (k contiguous) is
// read element by element with clamped indices -- what lands in the places past the end is never used (rows /
// columns past the edge are not stored, k past the end is zeroed in the ragged tile).
typedef double v2d_loose __attribute__((ext_vector_type(2), aligned(8)));

template <bool LOOSE> struct Mover {
  const double *src[VECS];
  long long step;
  int lds[VECS];  // index of element 0 of each vector inside a stage
  bool x_contig;
  bool lone[VECS];  // LOOSE, x contiguous: only the vector's first element (or none: src is clamped) lies inside the row

  // the vector's first k inside a k-tile
  static __device__ __forceinline__ int k_local(int v, bool xc) { return xc ? v >> 6 : ((v >> 4) & 7) * 2; }

  __device__ __forceinline__ void init(const double *base, long long s_x, long long s_k, int x0, int x_end, int k0,
                                       bool xc) {
    const int tid = threadIdx.x;
    x_contig = xc;
    step = (long long)BK * s_k;
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      const int v = tid + 256 * p, kl = k_local(v, xc);
      if (xc) {
        const int x = (v & 63) * 2;
        src[p] = base + (long long)(k0 + kl) * s_k + (LOOSE ? min(x0 + x, x_end - 1) : min(x0 + x, x_end - 2));
        lone[p] = x0 + x + 2 > x_end;
        lds[p] = kl * LD + x;
      } else {
        // lanes 0..15: 16 consecutive x of k-pair 0, lanes 16..31: the same x of k-pair 1, ...
        const int x = ((v >> 7) << 4) | (v & 15);
        src[p] = base + (long long)min(x0 + x, x_end - 1) * s_x + k0 + kl;
        lone[p] = false;
        lds[p] = kl * LD + x;
      }
    }
  }
  __device__ __forceinline__ void load(v2d (&r)[VECS]) {
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      r[p] = fetch(src[p], p);
      src[p] += step;
    }
  }
  // two consecutive elements from `at` (x contiguous: of a row, where the second may lie past its end)
  __device__ __forceinline__ v2d fetch(const double *at, int p) const {
    if constexpr (!LOOSE) return *reinterpret_cast<const v2d *>(at);
    else if (lone[p]) return v2d{at[0], at[0]};
    else return *reinterpret_cast<const v2d_loose *>(at);
  }
  // ragged last k-tile with kcount (< BK) valid k: vectors past the end re-read the last valid one
  __device__ __forceinline__ void load_ragged(v2d (&r)[VECS], long long s_k, int kcount) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      const int kl = k_local(tid + 256 * p, x_contig);
      if (LOOSE && !x_contig) {
        // elements are k = kl, kl + 1 of the tile; past the end, the last valid k instead
        r[p] = v2d{src[p][min(kl, kcount - 1) - kl], src[p][min(kl + 1, kcount - 1) - kl]};
      } else {
        const int back = max(kl - (kcount - (x_contig ? 1 : 2)), 0);
        r[p] = fetch(src[p] - (long long)back * s_k, p);
      }
      src[p] += step;
    }
  }
  __device__ __forceinline__ void store(const v2d (&r)[VECS], double *stage) const {
#pragma unroll
    for (int p = 0; p < VECS; ++p) {
      if (x_contig) {
        *reinterpret_cast<v2d *>(stage + lds[p]) = r[p];
      } else {
        stage[lds[p]] = r[p][0];
        stage[lds[p] + LD] = r[p][1];
      }
    }
  }
};

template <bool LOOSE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_mfma_f64_kernel(Problem p) {
  __shared__ Smem sm;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const double *A = reinterpret_cast<const double *>(p.A);
  const double *B = reinterpret_cast<const double *>(p.B);

  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;

  // byte offset, inside the LDS panel array, of this lane's operand for block 0 of k-quad 0
  int a_off = 8 * ((lane >> 4) * LD + wm * 64 + (lane & 15));
  int b_off = 8 * ((lane >> 4) * LD + wn * 64 + (lane & 15));

  v4d acc[4][4];
#pragma unroll
  for (int bi = 0; bi < 4; ++bi)
#pragma unroll
    for (int bj = 0; bj < 4; ++bj)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[bi][bj][r] = p.add_identity.f64;  // 0 for plus

  const int ntiles = (ke - kb + BK - 1) / BK;
  Mover<LOOSE> ma, mb;
  ma.init(A, p.sa_m, p.sa_k, m0, p.m, kb, a_xc);
  mb.init(B, p.sb_n, p.sb_k, n0, p.n, kb, b_xc);
  v2d ra[VECS], rb[VECS];
  auto fetch = [&](int k0) {
    const int kcount = ke - k0;
    if (kcount >= BK) {
      ma.load(ra);
      mb.load(rb);
    } else {
      ma.load_ragged(ra, p.sa_k, kcount);
      mb.load_ragged(rb, p.sb_k, kcount);
    }
  };
  if (ntiles > 0) {
    fetch(kb);
    ma.store(ra, &sm.a[0][0][0]);
    mb.store(rb, &sm.b[0][0][0]);
  }
  __syncthreads();

  int buf = 0, stage_step = BK * LD * 8;
  for (int t = 0; t < ntiles; ++t) {
    const int k0 = kb + t * BK;
    const bool more = t + 1 < ntiles;
    if (more) fetch(k0 + BK);
    __builtin_amdgcn_sched_barrier(0);
    // k past the end of a ragged last tile: its products must not count.  The
    // panels hold other data there, so those operands are replaced by zeros.
    const int kcount = min(BK, ke - k0);
    const char *pa = reinterpret_cast<const char *>(&sm.a[0][0][0]);
    const char *pb = reinterpret_cast<const char *>(&sm.b[0][0][0]);
#pragma unroll
    for (int kq = 0; kq < BK / 4; ++kq) {
      double av[4], bv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        av[q] = *reinterpret_cast<const double *>(pa + (kq * 4 * LD + q * 16) * 8 + a_off);
        bv[q] = *reinterpret_cast<const double *>(pb + (kq * 4 * LD + q * 16) * 8 + b_off);
      }
      if (kcount < BK) {
        const bool valid = kq * 4 + (lane >> 4) < kcount;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          av[q] = valid ? av[q] : 0.0;
          bv[q] = valid ? bv[q] : 0.0;
        }
      }
#pragma unroll
      for (int bi = 0; bi < 4; ++bi)
#pragma unroll
        for (int bj = 0; bj < 4; ++bj)
          acc[bi][bj] = __builtin_amdgcn_mfma_f64_16x16x4f64(av[bi], bv[bj], acc[bi][bj], 0, 0, 0);
      // the next tile's LDS stores go after the second of the four k-quads, under the matrix
      // instructions of the other two, instead of between the last of them and the barrier
      // (4096^3: 63.2 -> 65.4 TFLOP/s, 8192^3: 64.6 -> 67.0)
      if (kq == BK / 8 - 1) {
        __builtin_amdgcn_sched_barrier(0);
        if (more) {
          ma.store(ra, &sm.a[buf ^ 1][0][0]);
          mb.store(rb, &sm.b[buf ^ 1][0][0]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
    buf ^= 1;
    a_off += stage_step;
    b_off += stage_step;
    stage_step = -stage_step;
  }

  // ---- epilogue
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
#pragma unroll
  for (int bi = 0; bi < 4; ++bi)
#pragma unroll
    for (int bj = 0; bj < 4; ++bj) {
      const int col = n0 + wn * 64 + bj * 16 + (lane & 15);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + wm * 64 + bi * 16 + (lane >> 4) + 4 * r;
        if (row < p.m && col < p.n) {
          double v = acc[bi][bj][r];
          if (!partial) {
            v = alpha * v;
            if (source_needed) v = v + beta * C[(long long)row * p.ldc + col];
          }
          out[(long long)row * ld_out + col] = v;
        }
      }
    }
}

// the loads are 16-byte vectors: aligned bases, leading dimensions that are
// multiples of 2 and extents of at least one vector along the contiguous
// direction (so a clamped vector stays inside the matrix)
static bool can_run(const Problem &p) {
  auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;
  if (!al(p.A) || !al(p.B)) return false;
  if (a_xc ? (p.m % 2 || p.sa_k % 2) : (p.sa_k != 1 || p.k % 2 || p.sa_m % 2)) return false;
  if (b_xc ? (p.n % 2 || p.sb_k % 2) : (p.sb_k != 1 || p.k % 2 || p.sb_n % 2)) return false;
  return true;
}

// the element-aligned form asks for one contiguous direction per operand only
static bool loose_can_run(const Problem &p) { return (p.sa_m == 1 || p.sa_k == 1) && (p.sb_n == 1 || p.sb_k == 1); }

static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!loose_can_run(p)) return hipErrorNotSupported;
  const bool loose = !can_run(p);
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  // whole k-tiles, loadable straight into LDS: the hand-scheduled form of the same tile (faster at every size
  // measured, also where a round of workgroups is mostly empty: 2048^3 71.9 against 54.8 TFLOP/s)
  if (!loose && mfma_direct_f64_can_run(p)) return mfma_direct_f64_launch(p, s);
  if (p.batch > 1) return hipErrorNotSupported;  // the compiled kernel takes one product per launch
  dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1);
  if (loose) launch_kernel(gemm_mfma_f64_kernel<true>, grid, dim3(256), 0, s, p);
  else launch_kernel(gemm_mfma_f64_kernel<false>, grid, dim3(256), 0, s, p);
  return take_launch_status();
}

}  // namespace gemm_mfma_f64

launch_fn find_mfma_f64(int add_op, int mult_op) {
  if (add_op == kPlus && mult_op == kMultiplies) return gemm_mfma_f64::launch;
  return nullptr;
}

bool mfma_f64_can_run(const Problem &p) { return gemm_mfma_f64::loose_can_run(p); }

}  // namespace cuasr_amd
