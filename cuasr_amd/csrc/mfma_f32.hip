// Matrix-core assisted SRGEMM tiles for float.
//
// (1) min-plus / max-plus.  A tropical inner product needs one add and one
// min (or max) per term.  gfx950 has no packed-float min and this library
// does not use packed-float adds, so a vector-ALU-only kernel pays 1.5
// instructions per term.  Here the adds run on the matrix cores instead:
//
//     v_mfma_f32_32x32x2_f32 with  A = (a[i][k] | 1.0),  B = (1.0 | b[k][j]),  C = 0
//     gives  D[i][j] = a[i][k] * 1.0 + 1.0 * b[k][j] = fl(a[i][k] + b[k][j])
//
// for a whole 32x32 block of (i, j) at one k: multiplying by one is exact,
// adding zero is exact, and the remaining single addition is rounded once, to
// nearest even, like v_add_f32 (checked bit for bit on the device over random,
// denormal, huge and infinite operands by tests/test_gpu_mfma_add.py).  The
// vector ALU is left with one 3-input min/max per TWO terms
// (acc = min3(acc, t[k], t[k+1])), and runs concurrently with the matrix
// pipe.  The matrix pipe delivers 16 sums per clock per SIMD, the same rate
// as v_add_f32 alone, so the kernel is bound by the matrix pipe at
// 2 ops/lane/clock -- what a packed add + min3 kernel would reach at best.
//
// Replaces, for these two semirings, the reference's SIMT hierarchy
// (include/cuasr/gemm/threadblock/srmma_pipelined.h:153-288 down to
// include/cuasr/arch/srmma.h:84-91) and kernel body
// (include/cuasr/gemm/kernel/srgemm.h:156-321,
//  include/cuasr/gemm/kernel/srgemm_splitk_parallel.h:107-220).
//
// Layout: workgroup = 256 threads = 4 waves (2 x 2), output tile 128 x 128,
// wave tile 64 x 64 = 2 x 2 blocks of 32 x 32, k-tile 16.  LDS holds, per
// stage, A as [k/4][128 + 1] float4 (4 consecutive k of one row; entry 128 is
// (1,1,1,1)) and B likewise, so one ds_read_b128 per lane yields the operand
// registers of four k-steps: lanes 0..31 fetch their row, lanes 32..63 the
// ones entry (A), and the other way round for B.
#include "mfma_common.h"

namespace cuasr_amd {

namespace tropical {

using namespace mfma_panel;
constexpr int ROWS = BM + 1;  // + the ones entry

struct Smem {
  v4f a[2][KQ][ROWS];
  v4f b[2][KQ][ROWS];
};

template <bool IS_MIN> __device__ __forceinline__ float sel3(float acc, float x, float y) {
  return IS_MIN ? __builtin_fminf(__builtin_fminf(acc, x), y) : __builtin_fmaxf(__builtin_fmaxf(acc, x), y);
}
template <bool IS_MIN> __device__ __forceinline__ float sel2(float acc, float x) {
  return IS_MIN ? __builtin_fminf(acc, x) : __builtin_fmaxf(acc, x);
}

template <bool IS_MIN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void tropical_mfma_kernel(Problem p) {
  __shared__ Smem sm;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const float *A = reinterpret_cast<const float *>(p.A);
  const float *B = reinterpret_cast<const float *>(p.B);
  const float ident = p.add_identity.f32;

  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;

  // the ones entries never change
  if (tid < 2 * KQ) {
    const v4f ones = {1.0f, 1.0f, 1.0f, 1.0f};
    sm.a[tid / KQ][tid % KQ][BM] = ones;
    sm.b[tid / KQ][tid % KQ][BN] = ones;
  }

  // operand rows of this lane: A rows for lanes 0..31, the ones entry above;
  // B columns for lanes 32..63, the ones entry below
  int a_row[2], b_row[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    a_row[q] = lane < 32 ? wm * 64 + q * 32 + lane : BM;
    b_row[q] = lane < 32 ? BN : wn * 64 + q * 32 + (lane - 32);
  }

  v16f acc[2][2];
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bi][bj][r] = ident;

  const v16f zero = {0};
  const int ntiles = (ke - kb + BK - 1) / BK;
  v4f ra[2], rb[2];
  if (ntiles > 0) {
    load_panel(ra, A, p.sa_m, p.sa_k, m0, p.m, kb, ke, a_xc);
    load_panel(rb, B, p.sb_n, p.sb_k, n0, p.n, kb, ke, b_xc);
    store_panel<ROWS>(ra, sm.a[0], a_xc);
    store_panel<ROWS>(rb, sm.b[0], b_xc);
  }
  __syncthreads();

  // sums in flight between stages; they belong to block (1, 1), the block of
  // the last stage of a k-tile.  Starting them at the identity makes the very
  // first fold a no-op.
  v16f p0, p1;
#pragma unroll
  for (int r = 0; r < 16; ++r) p0[r] = p1[r] = ident;

  int buf = 0;
  for (int t = 0; t < ntiles; ++t) {
    const int k0 = kb + t * BK;
    const bool more = t + 1 < ntiles;
    if (more) {
      load_panel(ra, A, p.sa_m, p.sa_k, m0, p.m, k0 + BK, ke, a_xc);
      load_panel(rb, B, p.sb_n, p.sb_k, n0, p.n, k0 + BK, ke, b_xc);
    }
    const int kcount = min(BK, ke - k0);
    if (kcount == BK) {
      // 32 stages per k-tile: stage = (k-quad, k-pair, block).  Each stage
      // issues the two matrix instructions of its block and folds the sums of
      // the PREVIOUS stage into that stage's accumulators, so the vector ALU
      // works on finished results while the matrix pipe runs ahead.
      v4f af[2][2], bf[2][2];
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        af[0][q] = sm.a[buf][0][a_row[q]];
        bf[0][q] = sm.b[buf][0][b_row[q]];
      }
#pragma unroll
      for (int st = 0; st < 32; ++st) {
        const int kq = st >> 3, jp = (st >> 2) & 1, bi = (st >> 1) & 1, bj = st & 1, cur = kq & 1;
        const int pbi = ((st + 3) >> 1) & 1, pbj = (st + 3) & 1;  // block of the previous stage
        if ((st & 7) == 0 && kq + 1 < KQ) {
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            af[cur ^ 1][q] = sm.a[buf][kq + 1][a_row[q]];
            bf[cur ^ 1][q] = sm.b[buf][kq + 1][b_row[q]];
          }
        }
        const v16f n0 = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][bi][2 * jp], bf[cur][bj][2 * jp], zero, 0, 0, 0);
        const v16f n1 =
            __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][bi][2 * jp + 1], bf[cur][bj][2 * jp + 1], zero, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[pbi][pbj][r] = sel3<IS_MIN>(acc[pbi][pbj][r], p0[r], p1[r]);
        p0 = n0;
        p1 = n1;
        // keep the order "two matrix instructions, then the sixteen folds":
        // the folds read sums issued a whole stage earlier, which have left
        // the matrix pipe by the time this stage's second instruction is in
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      // ragged last k-tile: one k at a time, operands as single floats
#pragma unroll 1
      for (int kk = 0; kk < kcount; ++kk) {
        float av[2], bv[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          av[q] = reinterpret_cast<const float *>(&sm.a[buf][kk >> 2][a_row[q]])[kk & 3];
          bv[q] = reinterpret_cast<const float *>(&sm.b[buf][kk >> 2][b_row[q]])[kk & 3];
        }
#pragma unroll
        for (int bi = 0; bi < 2; ++bi)
#pragma unroll
          for (int bj = 0; bj < 2; ++bj) {
            const v16f t0 = __builtin_amdgcn_mfma_f32_32x32x2f32(av[bi], bv[bj], zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[bi][bj][r] = sel2<IS_MIN>(acc[bi][bj][r], t0[r]);
          }
      }
    }
    if (more) {
      store_panel<ROWS>(ra, sm.a[buf ^ 1], a_xc);
      store_panel<ROWS>(rb, sm.b[buf ^ 1], b_xc);
    }
    __syncthreads();
    buf ^= 1;
  }

#pragma unroll
  for (int r = 0; r < 16; ++r) acc[1][1][r] = sel3<IS_MIN>(acc[1][1][r], p0[r], p1[r]);

  // ---- epilogue.  Block (bi, bj), register r of lane l holds
  // row = 8*(r/4) + 4*(l/32) + r%4, column = l%32 of the 32 x 32 block.
  float *out;
  long long ld_out;
  const bool partial = p.workspace != nullptr;
  float alpha = 0.f, beta = 0.f;
  bool source_needed = false;
  if (partial) {
    out = reinterpret_cast<float *>(p.workspace) + (long long)blockIdx.y * p.m * p.n;
    ld_out = p.n;
  } else {
    out = reinterpret_cast<float *>(p.D);
    ld_out = p.ldd;
    const EpilogueScalars<float> e = resolve_scalars<float>(p, kPlus);
    alpha = e.alpha;
    beta = e.beta;
    source_needed = e.source_needed;
  }
  const float *C = reinterpret_cast<const float *>(p.C);
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj) {
      const int col = n0 + wn * 64 + bj * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 64 + bi * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        if (row < p.m && col < p.n) {
          float v = acc[bi][bj][r];
          if (!partial) {
            v = alpha + v;
            if (source_needed) v = sel2<IS_MIN>(v, beta + C[(long long)row * p.ldc + col]);
          }
          out[(long long)row * ld_out + col] = v;
        }
      }
    }
}

template <bool IS_MIN> static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!can_run(p)) return hipErrorNotSupported;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1);
  launch_kernel(tropical_mfma_kernel<IS_MIN>, grid, dim3(256), 0, s, p);
  return take_launch_status();
}

}  // namespace tropical

launch_fn find_mfma_gemm_f32(int add_op, int mult_op);

launch_fn find_mfma_f32(int add_op, int mult_op) {
  if (launch_fn f = find_mfma_gemm_f32(add_op, mult_op)) return f;
  if (mult_op == kPlus && add_op == kMinimum) return tropical::launch<true>;
  if (mult_op == kPlus && add_op == kMaximum) return tropical::launch<false>;
  return nullptr;
}

bool mfma_gemm_f32_can_run(const Problem &);
// (plus-times has an element-aligned form; the tropical tile needs 16-byte vectors)
bool mfma_f32_can_run(const Problem &p) {
  if (p.add_op == kPlus && p.mult_op == kMultiplies) return mfma_gemm_f32_can_run(p);
  return mfma_panel::can_run(p);
}

}  // namespace cuasr_amd
