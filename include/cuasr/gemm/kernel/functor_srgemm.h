// SRGEMM instantiated from arbitrary user functors -- the reference builds every kernel from whatever
// operator() the user writes (include/cuasr/arch/srmma.h:65-92 of the reference,
// examples/01_userdefined_semiring/userdefined_semiring.cu:56-99).  The library's tuned kernels cover the
// operators of cuasr/functional.h; a functor type that names none of them (no cuasr::op_tag
// specialisation) is compiled into this kernel instead, in the user's own translation unit, which
// therefore has to be compiled by hipcc.  The functors need a __host__ __device__ operator()(T, T) and
// the static members Identity and Annihilator, as in the reference.
//
// Results are those of the reference's host SRGEMM
// (tools/include/cuasr/reference/srgemm/host_srgemm.h:33-113) for ANY functor pair, associative or not:
// every output element is accumulated by one thread, accum = add(mult(a, b), accum) for k ascending from
// AddOp::Identity, then D = add(mult(alpha, accum), mult(beta, C)), or mult(alpha, accum) when the source
// is not needed (epilogue/thread/semiring_linear_combination.h:118-125, :152-183).  A product is never
// fused with the add that consumes it; what happens INSIDE a functor's own body follows the translation
// unit's -ffp-contract setting (hipcc by default fuses a*b+c on the device and not on the host: compile
// with -ffp-contract=off where a functor of that shape has to match a host run bit for bit).
//
//   workgroup 256 threads (16 x 16), output tile 64 x 64, thread tile 4 x 4, k-tile 16; panels staged
//   through LDS as [k][x]; operands addressed by element strides, so every layout and alignment runs.
#pragma once
#include <hip/hip_runtime.h>

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
};

// keeps the compiler from fusing a product into the add that follows it
template <typename T> __device__ __forceinline__ T functor_opaque(T v) {
  if constexpr (sizeof(T) == 4 || sizeof(T) == 8) asm volatile("" : "+v"(v));
  return v;
}

template <typename AddOp, typename MultOp, typename T>
__global__ __launch_bounds__(256) void functor_srgemm_kernel(FunctorSrgemmParams<T> p) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ T As[BK][BM + 4];
  __shared__ T Bs[BK][BN + 4];
  AddOp add_op;
  MultOp mult_op;
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int tiles_n = (p.n + BN - 1) / BN;
  const int m0 = (int)(blockIdx.x / tiles_n) * BM, n0 = (int)(blockIdx.x % tiles_n) * BN;

  T acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = AddOp::Identity;

  // a panel is 64 x 16 elements: four per thread, walked along whichever direction is contiguous in memory
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  for (int k0 = 0; k0 < p.k; k0 += BK) {
    const int kc = min(BK, p.k - k0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = tid + 256 * r;
      const int ax = a_kc ? e / BK : e % BM, ak = a_kc ? e % BK : e / BM;
      const int bx = b_kc ? e / BK : e % BN, bk = b_kc ? e % BK : e / BN;
      // rows, columns and k outside the problem read a valid element (clamped); they are never used
      const long long ai = min(m0 + ax, p.m - 1), akk = min(k0 + ak, p.k - 1);
      const long long bj = min(n0 + bx, p.n - 1), bkk = min(k0 + bk, p.k - 1);
      As[ak][ax] = p.A[ai * p.sa_m + akk * p.sa_k];
      Bs[bk][bx] = p.B[bkk * p.sb_k + bj * p.sb_n];
    }
    __syncthreads();
    for (int kk = 0; kk < kc; ++kk) {
      T a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = add_op(functor_opaque(mult_op(a[i], b[j])), acc[i][j]);
    }
    __syncthreads();
  }

  const T alpha = p.alpha_ptr ? *p.alpha_ptr : p.alpha, beta = p.beta_ptr ? *p.beta_ptr : p.beta;
  const bool source_needed = !(AddOp::Identity == mult_op(beta, MultOp::Identity));
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = m0 + ty * 4 + i;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + tx * 4 + j;
      if (row < p.m && col < p.n) {
        const T scaled = functor_opaque(mult_op(alpha, acc[i][j]));
        T out = scaled;
        if (source_needed) out = add_op(scaled, functor_opaque(mult_op(beta, p.C[row * p.sc_m + col * p.sc_n])));
        p.D[row * p.sd_m + col * p.sd_n] = out;
      }
    }
  }
}

/// Launch on `stream`; hipSuccess or the launch's error.
template <typename AddOp, typename MultOp, typename T>
inline hipError_t launch_functor_srgemm(FunctorSrgemmParams<T> const &p, hipStream_t stream) {
  if (p.m <= 0 || p.n <= 0) return hipSuccess;
  const long long tiles = (long long)((p.m + 63) / 64) * ((p.n + 63) / 64);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  void *args[] = {const_cast<void *>(static_cast<const void *>(&p))};
  return hipLaunchKernel(reinterpret_cast<const void *>(&functor_srgemm_kernel<AddOp, MultOp, T>), dim3((unsigned)tiles), dim3(256),
                         args, 0, stream);
}

}  // namespace kernel
}  // namespace gemm
}  // namespace cuasr
