// Second kernels of split-K for SRGEMMs built from arbitrary user functors: they fold the slices' raw
// accumulators (workspace[z][m][n], row-major, written by cuasr/gemm/kernel/functor_srgemm.h) and apply
// the epilogue, with the functors' own operator() -- one thread per 16-byte vector of a row.
//
//   functor_reduce_splitk_kernel   the parallel form, as the reference's ReduceSplitK
//       (include/cuasr/reduction/kernel/reduce_split_k.h:162-227, reduction/thread/reduction_operators.h:74-86):
//       acc = AddOp::Identity; acc = add(acc, workspace[z]) for z ascending (the accumulator is the LEFT
//       operand); source = C where the epilogue needs it, else AddOp::Identity; and ALWAYS the two-operand
//       epilogue D = add(mult(alpha, acc), mult(beta, source)).
//   functor_reduce_serial_kernel   the result of the reference's serial split-K
//       (include/cuasr/gemm/kernel/srgemm.h:249-320 with
//       epilogue/thread/semiring_linear_combination.h:129-134, :152-183) without its semaphores: the
//       slices' epilogues applied one after the other, slice 0 first with the caller's beta and C as
//       source, every later slice with beta = MultOp::Identity and the previous result as source; an
//       epilogue whose source is not needed is mult(alpha, acc) alone.
//
// Both write every element of D exactly once, after reading C at the same place: D may alias C.
#pragma once
#include <hip/hip_runtime.h>

#include "../../gemm/kernel/functor_srgemm.h"

namespace cuasr {
namespace reduction {
namespace kernel {

template <typename T> struct FunctorReduceParams {
  int m, n, slices;
  const T *workspace;
  const T *C; long long sc_m, sc_n;
  T *D;       long long sd_m, sd_n;
  T alpha, beta;
  const T *alpha_ptr, *beta_ptr;
};

template <typename AddOp, typename MultOp, typename T, bool SERIAL>
__global__ __launch_bounds__(256) void functor_reduce_kernel(FunctorReduceParams<T> p) {
  using gemm::kernel::functor_detail::opaque;
  constexpr int VW = 16 / sizeof(T);
  typedef T gvec_t __attribute__((ext_vector_type(VW), aligned(sizeof(T))));
  AddOp add_op;
  MultOp mult_op;
  const long long per_row = (p.n + VW - 1) / VW;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_row * p.m) return;
  const int row = (int)(idx / per_row), col = (int)(idx % per_row) * VW;
  const bool whole = col + VW <= p.n;
  const long long slice = (long long)p.m * p.n;
  const T *ws = p.workspace + (long long)row * p.n + col;
  const T alpha = p.alpha_ptr ? *p.alpha_ptr : p.alpha, beta = p.beta_ptr ? *p.beta_ptr : p.beta;
  const bool source_needed = !(AddOp::Identity == mult_op(beta, MultOp::Identity));

  auto load = [&](const T *src, T (&v)[VW]) {
    if (whole) {
      const gvec_t t = *reinterpret_cast<const gvec_t *>(src);
#pragma unroll
      for (int e = 0; e < VW; ++e) v[e] = t[e];
    } else {
#pragma unroll
      for (int e = 0; e < VW; ++e) v[e] = col + e < p.n ? src[e] : AddOp::Identity;
    }
  };
  T source[VW];
#pragma unroll
  for (int e = 0; e < VW; ++e) source[e] = AddOp::Identity;
  if (source_needed) {
#pragma unroll
    for (int e = 0; e < VW; ++e)
      if (col + e < p.n) source[e] = p.C[row * p.sc_m + (col + e) * p.sc_n];
  }

  T out[VW];
  if constexpr (!SERIAL) {
    T acc[VW];
#pragma unroll
    for (int e = 0; e < VW; ++e) acc[e] = AddOp::Identity;
    for (int z = 0; z < p.slices; ++z) {
      T w[VW];
      load(ws + z * slice, w);
#pragma unroll
      for (int e = 0; e < VW; ++e) acc[e] = add_op(acc[e], w[e]);
    }
#pragma unroll
    for (int e = 0; e < VW; ++e) out[e] = add_op(opaque(mult_op(alpha, acc[e])), opaque(mult_op(beta, source[e])));
  } else {
    // "source needed" as a later slice's epilogue sees it: its beta is MultOp::Identity
    const bool chain = !(AddOp::Identity == mult_op(MultOp::Identity, MultOp::Identity));
    T w[VW];
    load(ws, w);
#pragma unroll
    for (int e = 0; e < VW; ++e) {
      const T scaled = opaque(mult_op(alpha, w[e]));
      out[e] = source_needed ? add_op(scaled, opaque(mult_op(beta, source[e]))) : scaled;
    }
    for (int z = 1; z < p.slices; ++z) {
      load(ws + z * slice, w);
#pragma unroll
      for (int e = 0; e < VW; ++e) {
        const T scaled = opaque(mult_op(alpha, w[e]));
        out[e] = chain ? add_op(scaled, opaque(mult_op(MultOp::Identity, out[e]))) : scaled;
      }
    }
  }

  if (whole && p.sd_n == 1) {
    gvec_t o;
#pragma unroll
    for (int e = 0; e < VW; ++e) o[e] = out[e];
    *reinterpret_cast<gvec_t *>(p.D + row * p.sd_m + col) = o;
  } else {
#pragma unroll
    for (int e = 0; e < VW; ++e)
      if (col + e < p.n) p.D[row * p.sd_m + (col + e) * p.sd_n] = out[e];
  }
}

/// Launch on `stream`: serial = the ordered replay of the serial form's epilogues, else the parallel form's fold.
template <typename AddOp, typename MultOp, typename T>
inline hipError_t launch_functor_reduce(FunctorReduceParams<T> const &p, bool serial, hipStream_t stream) {
  if (p.m <= 0 || p.n <= 0) return hipSuccess;
  constexpr int VW = 16 / sizeof(T);
  const long long work = (long long)p.m * ((p.n + VW - 1) / VW);
  const long long groups = (work + 255) / 256;
  if (groups > 0x7fffffffLL) return hipErrorInvalidValue;
  void *args[] = {const_cast<void *>(static_cast<const void *>(&p))};
  const void *fn = serial ? reinterpret_cast<const void *>(&functor_reduce_kernel<AddOp, MultOp, T, true>)
                          : reinterpret_cast<const void *>(&functor_reduce_kernel<AddOp, MultOp, T, false>);
  return hipLaunchKernel(fn, dim3((unsigned)groups), dim3(256), args, 0, stream);
}

}  // namespace kernel
}  // namespace reduction
}  // namespace cuasr
