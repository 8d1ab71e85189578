// cuasr::Array<T, N> -- the fixed-size value array the reference's functors take besides scalars
// (cutlass::Array, pulled into the cuasr namespace at include/cuasr/functional.h:19 of the reference;
// used by the Array overloads of every functor, :52-79, and by user functors written against them,
// examples/01_userdefined_semiring/userdefined_semiring.cu:68-98).  The small subset those call sites
// use: element access, fill, size.  N elements of T, nothing else; trivially copyable.
#pragma once
#include <cstddef>

#if defined(__HIPCC__)
#define CUASR_HOST_DEVICE __host__ __device__
#else
#define CUASR_HOST_DEVICE
#endif

namespace cuasr {

template <typename T, int N> struct Array {
  using Element = T;
  using value_type = T;
  using reference = T &;
  using const_reference = T const &;
  static constexpr int kElements = N;
  static constexpr std::size_t kStorageElements = N;

  T storage[N];

  CUASR_HOST_DEVICE constexpr T &operator[](int i) { return storage[i]; }
  CUASR_HOST_DEVICE constexpr T const &operator[](int i) const { return storage[i]; }
  CUASR_HOST_DEVICE constexpr T &at(int i) { return storage[i]; }
  CUASR_HOST_DEVICE constexpr T const &at(int i) const { return storage[i]; }
  CUASR_HOST_DEVICE constexpr T *data() { return storage; }
  CUASR_HOST_DEVICE constexpr T const *data() const { return storage; }
  CUASR_HOST_DEVICE constexpr T *begin() { return storage; }
  CUASR_HOST_DEVICE constexpr T const *begin() const { return storage; }
  CUASR_HOST_DEVICE constexpr T *end() { return storage + N; }
  CUASR_HOST_DEVICE constexpr T const *end() const { return storage + N; }
  CUASR_HOST_DEVICE static constexpr int size() { return N; }
  CUASR_HOST_DEVICE static constexpr bool empty() { return N == 0; }
  CUASR_HOST_DEVICE constexpr void fill(T const &v) {
    for (int i = 0; i < N; ++i) storage[i] = v;
  }
  CUASR_HOST_DEVICE constexpr void clear() { fill(T()); }
};

}  // namespace cuasr
