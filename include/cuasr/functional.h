// Semiring operator functors of the cuASR API.
//
// Each functor has the reference's scalar semantics and constants
// (include/cuasr/functional.h:28-36, :39-283 of the reference):
//   plus        l + r           Identity 0,      Annihilator max()
//   multiplies  l * r           Identity 1,      Annihilator 0
//   minimum     r < l ? r : l   Identity max(),  Annihilator min()
//   maximum     l < r ? r : l   Identity min(),  Annihilator max()
//   binary_and  l && r (0/1)    Identity 1,      Annihilator 0
//   binary_or   l || r (0/1)    Identity 0,      Annihilator 1
// where max()/min() are std::numeric_limits<T>::max()/min() -- for floating
// point min() is the smallest positive normal, exactly as in the reference.
// Added here: binary_xor (the reference's user-defined example,
// examples/01_userdefined_semiring/userdefined_semiring.cu:56-66), bitwise
// and/or for bit-packed words, and cuasr::inf::minimum / maximum / plus whose
// constants are true infinities (what shortest-path data with unreachable
// pairs needs).
//
// The library's tuned kernels are not instantiated from these functors; a functor
// type maps to an operator tag of the C ABI through cuasr::op_tag<Functor>, which
// user code can specialise for its own functor types (see binary_xor below).  A
// functor type that is none of these operators gets a kernel built from its
// operator() (cuasr/gemm/kernel/functor_srgemm.h), as in the reference.
#pragma once
#include <limits>

#include "array.h"
#include "types.h"

namespace cuasr {

/// Which operator of the C ABI a functor type is.  Specialise it for a functor of your own that computes one
/// of those operators (as binary_xor below); a functor type without a specialisation counts as "none of
/// them" (value < 0): device::Srgemm then builds its kernel from the functor's operator() itself, which
/// needs the translation unit to be compiled by hipcc (cuasr/gemm/kernel/functor_srgemm.h).
template <typename F> struct op_tag { static int const value = -1; };

namespace detail {
template <typename T> constexpr T highest() { return std::numeric_limits<T>::max(); }
template <typename T> constexpr T lowest_ref() { return std::numeric_limits<T>::min(); }  // sic: the reference's "-inf"
template <typename T> constexpr T pos_inf() {
  return std::numeric_limits<T>::has_infinity ? std::numeric_limits<T>::infinity() : std::numeric_limits<T>::max();
}
template <typename T> constexpr T neg_inf() {
  return std::numeric_limits<T>::has_infinity ? -std::numeric_limits<T>::infinity() : std::numeric_limits<T>::lowest();
}
}  // namespace detail

// Besides the scalar form every functor has the reference's three element-wise forms on Array<T, N>
// (functional.h:52-79 and the same three per functor): array with array, array with scalar, scalar with array.
#define CUASR_AMD_FUNCTOR(NAME, IDENT, ANNIH, EXPR)                               \
  template <typename T, int N = 1> struct NAME {                                  \
    static constexpr T Identity = IDENT;                                          \
    static constexpr T Annihilator = ANNIH;                                       \
    CUASR_HOST_DEVICE constexpr T operator()(T lhs, T const &rhs) const { return EXPR; } \
    CUASR_HOST_DEVICE constexpr Array<T, N> operator()(Array<T, N> const &lhs, Array<T, N> const &rhs) const { \
      Array<T, N> result{};                                                       \
      for (int i = 0; i < N; ++i) result[i] = (*this)(lhs[i], rhs[i]);            \
      return result;                                                              \
    }                                                                             \
    CUASR_HOST_DEVICE constexpr Array<T, N> operator()(Array<T, N> const &lhs, T const &scalar) const { \
      Array<T, N> result{};                                                       \
      for (int i = 0; i < N; ++i) result[i] = (*this)(lhs[i], scalar);            \
      return result;                                                              \
    }                                                                             \
    CUASR_HOST_DEVICE constexpr Array<T, N> operator()(T const &scalar, Array<T, N> const &rhs) const { \
      Array<T, N> result{};                                                       \
      for (int i = 0; i < N; ++i) result[i] = (*this)(scalar, rhs[i]);            \
      return result;                                                              \
    }                                                                             \
  };                                                                              \
  template <typename T, int N> constexpr T NAME<T, N>::Identity;                  \
  template <typename T, int N> constexpr T NAME<T, N>::Annihilator;
#define CUASR_AMD_OP_TAG(NAME, TAG) \
  template <typename T, int N> struct op_tag<NAME<T, N>> { static int const value = TAG; };

CUASR_AMD_FUNCTOR(plus, static_cast<T>(0), detail::highest<T>(), static_cast<T>(lhs + rhs))
CUASR_AMD_FUNCTOR(multiplies, static_cast<T>(1), static_cast<T>(0), static_cast<T>(lhs * rhs))
CUASR_AMD_FUNCTOR(minimum, detail::highest<T>(), detail::lowest_ref<T>(), (rhs < lhs ? rhs : lhs))
CUASR_AMD_FUNCTOR(maximum, detail::lowest_ref<T>(), detail::highest<T>(), (lhs < rhs ? rhs : lhs))
CUASR_AMD_FUNCTOR(binary_and, static_cast<T>(true), static_cast<T>(false), static_cast<T>(lhs && rhs))
CUASR_AMD_FUNCTOR(binary_or, static_cast<T>(false), static_cast<T>(true), static_cast<T>(lhs || rhs))
CUASR_AMD_FUNCTOR(binary_xor, static_cast<T>(0), static_cast<T>(0), static_cast<T>(lhs ^ rhs))
CUASR_AMD_FUNCTOR(bitwise_and, static_cast<T>(~static_cast<T>(0)), static_cast<T>(0), static_cast<T>(lhs & rhs))
CUASR_AMD_FUNCTOR(bitwise_or, static_cast<T>(0), static_cast<T>(~static_cast<T>(0)), static_cast<T>(lhs | rhs))

CUASR_AMD_OP_TAG(plus, CUASR_AMD_OP_PLUS)
CUASR_AMD_OP_TAG(multiplies, CUASR_AMD_OP_MULTIPLIES)
CUASR_AMD_OP_TAG(minimum, CUASR_AMD_OP_MINIMUM)
CUASR_AMD_OP_TAG(maximum, CUASR_AMD_OP_MAXIMUM)
CUASR_AMD_OP_TAG(binary_and, CUASR_AMD_OP_LOGICAL_AND)
CUASR_AMD_OP_TAG(binary_or, CUASR_AMD_OP_LOGICAL_OR)
CUASR_AMD_OP_TAG(binary_xor, CUASR_AMD_OP_BIT_XOR)
CUASR_AMD_OP_TAG(bitwise_and, CUASR_AMD_OP_BIT_AND)
CUASR_AMD_OP_TAG(bitwise_or, CUASR_AMD_OP_BIT_OR)

/// The same operators with true infinities as their constants.
namespace inf {
CUASR_AMD_FUNCTOR(plus, static_cast<T>(0), detail::pos_inf<T>(), static_cast<T>(lhs + rhs))
CUASR_AMD_FUNCTOR(minimum, detail::pos_inf<T>(), detail::neg_inf<T>(), (rhs < lhs ? rhs : lhs))
CUASR_AMD_FUNCTOR(maximum, detail::neg_inf<T>(), detail::pos_inf<T>(), (lhs < rhs ? rhs : lhs))
/// plus as the multiplication of a max-semiring: its zero is -inf
CUASR_AMD_FUNCTOR(plus_for_max, static_cast<T>(0), detail::neg_inf<T>(), static_cast<T>(lhs + rhs))
}  // namespace inf

CUASR_AMD_OP_TAG(inf::plus, CUASR_AMD_OP_PLUS)
CUASR_AMD_OP_TAG(inf::minimum, CUASR_AMD_OP_MINIMUM)
CUASR_AMD_OP_TAG(inf::maximum, CUASR_AMD_OP_MAXIMUM)
CUASR_AMD_OP_TAG(inf::plus_for_max, CUASR_AMD_OP_PLUS)

}  // namespace cuasr
