// plus-times ("control") semiring for float on the matrix cores:
//     D = alpha * (A . B) + beta * C      with v_mfma_f32_32x32x2_f32
//
// The only semiring a matrix instruction computes as is.  Replaces, for this
// pair, the reference's SIMT kernel (include/cuasr/gemm/kernel/srgemm.h:156-321
// with DefaultSemiRingConfiguration<plus, multiplies>,
// include/cuasr/gemm/device/default_srgemm_configuration.h:44-72).  The sum over
// k is formed in the instruction's order (pairs of k, fused multiply-adds), not
// the host reference's strictly sequential unfused order, so results agree with
// it to rounding -- |d - r| <= 1e-5 * sum_k |a||b| -- not bit for bit; the
// vector-ALU tile (kernel = VALU / VALU_DIRECT) stays available for a bit-exact
// plus-times.
//
// Workgroup 256 threads = 4 waves (2 x 2), output tile 128 x 128, wave tile
// 64 x 64 = 2 x 2 blocks of 32 x 32 (64 accumulator registers), k-tile 16.
// LDS per stage: A and B as [k/4][128][4] (4 consecutive k of one row/column
// per 16 bytes).  The instruction wants k = 2q from lanes 0..31 and k = 2q + 1
// from lanes 32..63, so a lane reads the two floats (k, k + 2) at its row, the
// upper half-wave one float further along: one ds_read2_b32 per block row per
// k-quad feeds two matrix instructions.
#include "mfma_common.h"

namespace cuasr_amd {
namespace gemm_mfma {

using namespace mfma_panel;

struct Smem {
  v4f a[2][KQ][BM];
  v4f b[2][KQ][BN];
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_mfma_kernel(Problem p) {
  __shared__ Smem sm;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const float *A = reinterpret_cast<const float *>(p.A);
  const float *B = reinterpret_cast<const float *>(p.B);

  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;

  // float index, inside one k-quad of a stage, of this lane's operand pair
  int a_idx[2], b_idx[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    a_idx[q] = (wm * 64 + q * 32 + (lane & 31)) * 4 + (lane >> 5);
    b_idx[q] = (wn * 64 + q * 32 + (lane & 31)) * 4 + (lane >> 5);
  }

  v16f acc[2][2];
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bi][bj][r] = p.add_identity.f32;  // 0 for plus

  const int ntiles = (ke - kb + BK - 1) / BK;
  v4f ra[2], rb[2];
  if (ntiles > 0) {
    load_panel(ra, A, p.sa_m, p.sa_k, m0, p.m, kb, ke, a_xc);
    load_panel(rb, B, p.sb_n, p.sb_k, n0, p.n, kb, ke, b_xc);
    store_panel<BM>(ra, sm.a[0], a_xc);
    store_panel<BN>(rb, sm.b[0], b_xc);
  }
  __syncthreads();

  int buf = 0;
  for (int t = 0; t < ntiles; ++t) {
    const int k0 = kb + t * BK;
    const bool more = t + 1 < ntiles;
    if (more) {
      load_panel(ra, A, p.sa_m, p.sa_k, m0, p.m, k0 + BK, ke, a_xc);
      load_panel(rb, B, p.sb_n, p.sb_k, n0, p.n, k0 + BK, ke, b_xc);
    }
    // k past the end of a ragged last tile: its products must not count.  The
    // panels hold clamped (finite or not) data there, so the operands of those
    // k are replaced by zeros: 0 * 0 adds nothing.
    const int kcount = min(BK, ke - k0);
    const float *pa = reinterpret_cast<const float *>(&sm.a[buf][0][0]);
    const float *pb = reinterpret_cast<const float *>(&sm.b[buf][0][0]);
#pragma unroll
    for (int kq = 0; kq < KQ; ++kq) {
      float av[2][2], bv[2][2];  // [block][k-pair of the quad]
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        av[q][0] = pa[kq * BM * 4 + a_idx[q]];
        av[q][1] = pa[kq * BM * 4 + a_idx[q] + 2];
        bv[q][0] = pb[kq * BN * 4 + b_idx[q]];
        bv[q][1] = pb[kq * BN * 4 + b_idx[q] + 2];
      }
      if (kcount < BK) {
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const bool valid = kq * 4 + 2 * j + (lane >> 5) < kcount;
            av[q][j] = valid ? av[q][j] : 0.0f;
            bv[q][j] = valid ? bv[q][j] : 0.0f;
          }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi)
#pragma unroll
          for (int bj = 0; bj < 2; ++bj)
            acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[bi][j], bv[bj][j], acc[bi][bj], 0, 0, 0);
    }
    if (more) {
      store_panel<BM>(ra, sm.a[buf ^ 1], a_xc);
      store_panel<BN>(rb, sm.b[buf ^ 1], b_xc);
    }
    __syncthreads();
    buf ^= 1;
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
            v = alpha * v;
            if (source_needed) v = v + beta * C[(long long)row * p.ldc + col];
          }
          out[(long long)row * ld_out + col] = v;
        }
      }
    }
}

static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!can_run(p)) return hipErrorNotSupported;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1);
  hipLaunchKernelGGL(gemm_mfma_kernel, grid, dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace gemm_mfma

launch_fn find_mfma_gemm_f32(int add_op, int mult_op) {
  if (add_op == kPlus && mult_op == kMultiplies) return gemm_mfma::launch;
  return nullptr;
}

}  // namespace cuasr_amd
