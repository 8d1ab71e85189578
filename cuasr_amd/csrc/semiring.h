// Device-side scalar operators of the semirings and the shared problem record.
//
// Operator semantics are those of the reference functors
// (include/cuasr/functional.h:46-49, :89-92, :132, :172, :212, :252 and
// examples/01_userdefined_semiring/userdefined_semiring.cu:56-66): minimum and
// maximum return one of their operands, logical and/or return 0 or 1, the
// bitwise forms exist for integer element types only.  For floating point the
// min/max forms map to the hardware min/max instructions, which agree with the
// reference's comparisons for every input that is not a NaN and not a tie
// between +0 and -0.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <tuple>
#include <type_traits>
#include <utility>

#include "../../include/cuasr_amd.h"

namespace cuasr_amd {

enum : int { kPlus = 0, kMultiplies = 1, kMinimum = 2, kMaximum = 3, kLogicalAnd = 4,
             kLogicalOr = 5, kBitAnd = 6, kBitOr = 7, kBitXor = 8 };

typedef _Float16 half_t;  // IEEE binary16; arithmetic on it rounds every result to binary16

template <typename T> struct is_fp : std::integral_constant<bool, std::is_floating_point<T>::value> {};
template <> struct is_fp<half_t> : std::true_type {};

template <typename T> __device__ __forceinline__ T hw_min(T l, T r) { return r < l ? r : l; }
template <typename T> __device__ __forceinline__ T hw_max(T l, T r) { return l < r ? r : l; }
template <> __device__ __forceinline__ float hw_min<float>(float l, float r) { return __builtin_fminf(l, r); }
template <> __device__ __forceinline__ float hw_max<float>(float l, float r) { return __builtin_fmaxf(l, r); }
template <> __device__ __forceinline__ double hw_min<double>(double l, double r) { return __builtin_fmin(l, r); }
template <> __device__ __forceinline__ double hw_max<double>(double l, double r) { return __builtin_fmax(l, r); }

// Compile-time operator.
//   Op<OP>::apply(l, r)   fast form: floating-point min/max are the hardware
//                         instructions (order-free, one instruction)
//   Op<OP>::strict(l, r)  the reference's comparison, operand order included:
//                         minimum = rhs < lhs ? rhs : lhs, maximum = lhs < rhs ? rhs : lhs
// The two differ only when the operands are +0 and -0 (or NaN).  Sums, minima
// and maxima of data free of -0 never produce -0; products do (0 * negative),
// so kernels use the strict form wherever `multiplies` feeds a min or max.
// What the logical operators ask of an operand: is it anything but zero?  +0 and -0 are false, NaN is true
// (functional.h:212, :252 convert to bool).  Floating point is asked by its bit pattern, and the pattern passes
// through an empty asm statement: the compiler recognises the integer test of a bit-cast float as a floating-point
// comparison, and in a translation unit that lets it assume NaN-free data it then picks the ordered one (NaN false).
template <typename T> __device__ __forceinline__ bool truth(T x) {
  if constexpr (is_fp<T>::value) {
    typedef typename std::conditional<sizeof(T) == 8, uint64_t, typename std::conditional<sizeof(T) == 4, uint32_t, uint16_t>::type>::type bits_t;
    typedef typename std::conditional<sizeof(T) == 8, uint64_t, uint32_t>::type reg_t;
    reg_t bits = __builtin_bit_cast(bits_t, x);
    asm("" : "+v"(bits));
    return reg_t(bits << (sizeof(T) == 2 ? 17 : 1)) != 0;
  } else {
    return x != T(0);
  }
}

template <int OP> struct Op {
  template <typename T> static __device__ __forceinline__ T strict(T l, T r) {
    if constexpr (std::is_same<T, half_t>::value && (OP == kMinimum || OP == kMaximum)) {
      // binary16: compared and chosen as integers (sign-magnitude to two's complement, so +0 and -0 tie), because
      // the compiler turns the floating-point form of this comparison into the min / max instruction, which
      // returns -0 for that tie whatever the operand order.  (NaN-free data, as everywhere on the fast paths.)
      const unsigned short rb = __builtin_bit_cast(unsigned short, r), lb = __builtin_bit_cast(unsigned short, l);
      const int rk = (rb & 0x8000) ? -(int)(rb & 0x7fff) : (int)(rb & 0x7fff);
      const int lk = (lb & 0x8000) ? -(int)(lb & 0x7fff) : (int)(lb & 0x7fff);
      const bool take_r = OP == kMinimum ? rk < lk : lk < rk;
      return __builtin_bit_cast(half_t, (unsigned short)(take_r ? rb : lb));
    } else if constexpr (is_fp<T>::value && (OP == kMinimum || OP == kMaximum)) {
      // float, double: the operand the comparison may pick passes through an empty asm statement.  Written plainly,
      // in a translation unit that assumes NaN-free data the compiler turns compare-and-select into the min / max
      // instruction, which returns -0 for a +0 / -0 tie whatever the operand order (min(+0, 0 * C) with C < 0 then
      // comes out as -0 where the reference keeps the left operand).
      T picked = r;
      asm("" : "+v"(picked));
      return (OP == kMinimum ? r < l : l < r) ? picked : l;
    } else if constexpr (OP == kMinimum) return r < l ? r : l;
    else if constexpr (OP == kMaximum) return l < r ? r : l;
    else return apply(l, r);
  }
  template <typename T> static __device__ __forceinline__ T apply(T l, T r) {
    if constexpr (OP == kPlus) return l + r;
    else if constexpr (OP == kMultiplies) return l * r;
    else if constexpr (OP == kMinimum) return hw_min<T>(l, r);
    else if constexpr (OP == kMaximum) return hw_max<T>(l, r);
    else if constexpr (OP == kLogicalAnd) return T(truth(l) && truth(r));
    else if constexpr (OP == kLogicalOr) return T(truth(l) || truth(r));
    else if constexpr (!is_fp<T>::value) {
      if constexpr (OP == kBitAnd) return l & r;
      else if constexpr (OP == kBitOr) return l | r;
      else return l ^ r;
    } else {
      return l;  // bitwise on floating point is rejected on the host
    }
  }
};

// Run-time operator with the strict semantics (naive kernel, reduction, scalars)
template <typename T> __device__ __forceinline__ T apply_op(int op, T l, T r) {
  switch (op) {
    case kPlus: return Op<kPlus>::strict(l, r);
    case kMultiplies: return Op<kMultiplies>::strict(l, r);
    case kMinimum: return Op<kMinimum>::strict(l, r);
    case kMaximum: return Op<kMaximum>::strict(l, r);
    case kLogicalAnd: return Op<kLogicalAnd>::strict(l, r);
    case kLogicalOr: return Op<kLogicalOr>::strict(l, r);
    case kBitAnd: return Op<kBitAnd>::strict(l, r);
    case kBitOr: return Op<kBitOr>::strict(l, r);
    default: return Op<kBitXor>::strict(l, r);
  }
}

// add(prod, acc) in the host reference's operand order
// (tools/include/cuasr/reference/srgemm/host_srgemm.h:87), strict when a
// product can be -0 and the add is a comparison
template <int ADD, int MUL, typename T> __device__ __forceinline__ T fold(T prod, T acc) {
  if constexpr ((ADD == kMinimum || ADD == kMaximum) && MUL == kMultiplies && is_fp<T>::value) return Op<ADD>::strict(prod, acc);
  else return Op<ADD>::apply(acc, prod);
}

// One term of the inner product, acc <- add(mult(a, b), acc).  For xor-and and or-and on 32-bit
// words gfx950's three-input bit operation does the whole term in one instruction, and that
// instruction issues almost as fast as a two-input one (per wave: v_and_b32 and v_xor_b32 2.1
// cycles each, v_bitop3_b32 2.6, v_and_or_b32 4.2).  The table is the function's value on
// a = 0xF0, b = 0xCC, acc = 0xAA.
template <int ADD, int MUL, typename T> struct fused_bit_term
    : std::integral_constant<bool, sizeof(T) == 4 && !is_fp<T>::value && MUL == kBitAnd && (ADD == kBitXor || ADD == kBitOr)> {};
__device__ __forceinline__ uint32_t xor_and_term(uint32_t acc, uint32_t a, uint32_t b) {
  return __builtin_amdgcn_bitop3_b32(a, b, acc, 0x6a);  // acc ^ (a & b)
}
__device__ __forceinline__ uint32_t or_and_term(uint32_t acc, uint32_t a, uint32_t b) {
  return __builtin_amdgcn_bitop3_b32(a, b, acc, 0xea);  // acc | (a & b)
}
template <int ADD, int MUL, typename T> __device__ __forceinline__ T term(T acc, T a, T b) {
  if constexpr (fused_bit_term<ADD, MUL, T>::value) {
    if constexpr (ADD == kBitXor) return T(xor_and_term(uint32_t(acc), uint32_t(a), uint32_t(b)));
    else return T(or_and_term(uint32_t(acc), uint32_t(a), uint32_t(b)));
  } else {
    return fold<ADD, MUL>(Op<MUL>::apply(a, b), acc);
  }
}

// add(lhs, rhs) of the epilogue, D = add(mult(alpha, acc), mult(beta, C)), same rule
template <int ADD, int MUL, typename T> __device__ __forceinline__ T fold_epilogue(T lhs, T rhs) {
  if constexpr ((ADD == kMinimum || ADD == kMaximum) && MUL == kMultiplies && is_fp<T>::value) return Op<ADD>::strict(lhs, rhs);
  else return Op<ADD>::apply(lhs, rhs);
}

template <typename T> __host__ __device__ __forceinline__ T scalar_as(const cuasr_amd_scalar &s);
template <> __host__ __device__ __forceinline__ float scalar_as<float>(const cuasr_amd_scalar &s) { return s.f32; }
template <> __host__ __device__ __forceinline__ double scalar_as<double>(const cuasr_amd_scalar &s) { return s.f64; }
template <> __host__ __device__ __forceinline__ int32_t scalar_as<int32_t>(const cuasr_amd_scalar &s) { return s.i32; }
template <> __host__ __device__ __forceinline__ uint32_t scalar_as<uint32_t>(const cuasr_amd_scalar &s) { return s.u32; }
template <> __host__ __device__ __forceinline__ half_t scalar_as<half_t>(const cuasr_amd_scalar &s) {
  return __builtin_bit_cast(half_t, s.f16);
}

// add(v, *addr) into *addr, atomically at device scope and without waiting for an answer, for the adds that have a
// native atomic on 4-byte elements: minimum and maximum (integers directly; floats through the integer atomics --
// a float without sign bit orders like its bits as a signed integer, one with sign bit the other way round like its
// bits as an unsigned integer, and every float of the second kind is below every float of the first both as a number
// and as a signed integer / above as an unsigned one), or and xor on words.  NaN-free data, as everywhere the
// hardware minimum is used; the results do not depend on the order in which the folds arrive.
template <typename T, int ADD> struct has_native_fold
    : std::integral_constant<bool, sizeof(T) == 4 && (ADD == kMinimum || ADD == kMaximum || (!is_fp<T>::value && (ADD == kBitOr || ADD == kBitXor)))> {};

template <int ADD, typename T> __device__ __forceinline__ void native_fold(T *addr, T v) {
  static_assert(has_native_fold<T, ADD>::value, "no native atomic for this add on this element type");
  const int bits = __builtin_bit_cast(int, v);
  int *si = reinterpret_cast<int *>(addr);
  unsigned *ui = reinterpret_cast<unsigned *>(addr);
  if constexpr (ADD == kBitXor) {
    __hip_atomic_fetch_xor(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else if constexpr (ADD == kBitOr) {
    __hip_atomic_fetch_or(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else if constexpr (is_fp<T>::value) {
    if constexpr (ADD == kMinimum) {
      if (bits >= 0) __hip_atomic_fetch_min(si, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_fetch_max(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      if (bits >= 0) __hip_atomic_fetch_max(si, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      else __hip_atomic_fetch_min(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else if constexpr (std::is_signed<T>::value) {
    if constexpr (ADD == kMinimum) __hip_atomic_fetch_min(si, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else __hip_atomic_fetch_max(si, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  } else {
    if constexpr (ADD == kMinimum) __hip_atomic_fetch_min(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else __hip_atomic_fetch_max(ui, (unsigned)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// The problem in kernel form.  The host has already turned a column-major C
// into the transposed problem (C^T = B^T (x) A^T, as the reference does in
// include/cuasr/gemm/device/srgemm.h:432-453, :513-523), so C and D are always
// row-major here and A, B are addressed by element strides.
struct Problem {
  int m, n, k;
  const void *A; long long sa_m, sa_k;   // A[i][kk] at A + i*sa_m + kk*sa_k
  const void *B; long long sb_k, sb_n;   // B[kk][j] at B + kk*sb_k + j*sb_n
  const void *C; long long ldc;          // C[i][j] at C + i*ldc + j
  void *D;       long long ldd;
  cuasr_amd_scalar alpha, beta, add_identity, mult_identity;
  const void *alpha_ptr, *beta_ptr;
  int add_op, mult_op;
  // split-K: slice z covers k in [z*k_per_slice, min(k, (z+1)*k_per_slice));
  // partial accumulators go to workspace[z][m][n] (row-major, ld = n)
  int slices, k_per_slice;
  void *workspace;
  // split-K of a small output on the staged tiles: every slice's k range is shared out over k_sub workgroups
  // (blockIdx.y = slice * k_sub + part), which fold their accumulators into the slice's partial tile with one
  // atomic per element; the host fills the workspace with the additive identity first.  0 or 1: one workgroup
  // per tile and slice, plain stores.
  int k_sub;
  // strided batch (tile kernels only): product blockIdx.z works on A, B, C, D moved on by z times
  // these element strides; batch = 1 for a single product
  int batch;
  long long batch_a, batch_b, batch_c, batch_d;
};

// the operands of product blockIdx.z of a strided batch
template <typename T, typename TI = T> __device__ __forceinline__ void select_batch(Problem &p) {
  if (p.batch > 1) {
    const long long z = blockIdx.z;
    p.A = reinterpret_cast<const TI *>(p.A) + z * p.batch_a;
    p.B = reinterpret_cast<const TI *>(p.B) + z * p.batch_b;
    if (p.C) p.C = reinterpret_cast<const T *>(p.C) + z * p.batch_c;
    p.D = reinterpret_cast<T *>(p.D) + z * p.batch_d;
  }
}

// Epilogue scalars resolved on the device (alpha/beta may live in device memory).
template <typename T> struct EpilogueScalars {
  T alpha, beta, ident;
  bool source_needed;
};

template <typename T> __device__ __forceinline__ EpilogueScalars<T> resolve_scalars(const Problem &p, int mult_op) {
  EpilogueScalars<T> e;
  e.alpha = p.alpha_ptr ? *reinterpret_cast<const T *>(p.alpha_ptr) : scalar_as<T>(p.alpha);
  e.beta = p.beta_ptr ? *reinterpret_cast<const T *>(p.beta_ptr) : scalar_as<T>(p.beta);
  e.ident = scalar_as<T>(p.add_identity);
  // source needed <=> add_identity != mult(beta, mult_identity)
  // (epilogue/thread/semiring_linear_combination.h:118-125)
  e.source_needed = e.ident != apply_op<T>(mult_op, e.beta, scalar_as<T>(p.mult_identity));
  return e;
}

// Tile order of the stream-K launches (the kernel and the launch that prepares D must agree on it): down
// the columns of a band of 8 tile rows, so that workgroups with neighbouring ids share panels.
__host__ __device__ __forceinline__ void streamk_tile_coords(long long tile, int tiles_m, int tiles_n, int &bm, int &bn) {
  const int band = (int)(tile / (8LL * tiles_n)), in_band = (int)(tile - (long long)band * 8 * tiles_n);
  const int rows = tiles_m - band * 8 < 8 ? tiles_m - band * 8 : 8;
  bm = band * 8 + in_band % rows;
  bn = in_band / rows;
}

typedef hipError_t (*launch_fn)(const Problem &, hipStream_t);

// Kernel launches report the launch call's own status.  (hipGetLastError() after a launch would also
// return -- and clear -- an error some earlier call of the CALLER left behind on this thread, e.g. the
// hipErrorNotReady of a stream query: a good launch would read as a failure and the caller's error be lost.)
// launch_kernel records the first failure of the calling thread; take_launch_status returns and clears it.
inline thread_local hipError_t launch_status_ = hipSuccess;
template <typename... P, size_t... I>
inline hipError_t launch_packed_(const void *kernel, dim3 grid, dim3 block, size_t shmem, hipStream_t s, std::tuple<P...> &params,
                                 std::index_sequence<I...>) {
  void *ptrs[] = {static_cast<void *>(&std::get<I>(params))...};
  return hipLaunchKernel(kernel, grid, block, ptrs, shmem, s);
}
template <typename... P, typename... A>
inline void launch_kernel(void (*kernel)(P...), dim3 grid, dim3 block, size_t shmem, hipStream_t s, A &&...args) {
  static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
  std::tuple<P...> params{static_cast<P>(args)...};
  const hipError_t e = launch_packed_(reinterpret_cast<const void *>(kernel), grid, block, shmem, s, params, std::index_sequence_for<P...>{});
  if (e != hipSuccess && launch_status_ == hipSuccess) launch_status_ = e;
}
inline hipError_t take_launch_status() {
  const hipError_t e = launch_status_;
  launch_status_ = hipSuccess;
  return e;
}

// kernel-family lookups, one definition per translation unit that owns them
launch_fn find_naive(int dtype);
launch_fn find_valu(int dtype, int add_op, int mult_op);
launch_fn find_mfma(int dtype, int add_op, int mult_op);
launch_fn find_reduce(int dtype);
launch_fn find_reduce_serial(int dtype);
// the stream-K form of the direct tile: (problem, workgroups, stream), and the launch before it that writes the
// source term into the output tiles the workgroups share: (problem, tile rows, tile columns, first shared tile, stream)
typedef hipError_t (*streamk_fn)(const Problem &, int, hipStream_t);
typedef hipError_t (*prepare_fold_fn)(const Problem &, int, int, long long, hipStream_t);
prepare_fold_fn find_prepare_fold(int dtype);

}  // namespace cuasr_amd
