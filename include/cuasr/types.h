// Value types of the cuASR-compatible operator API: status codes, problem
// coordinates, layouts and tensor references.  The reference takes these from
// CUTLASS (cutlass::Status, cutlass::gemm::GemmCoord, cutlass::MatrixCoord,
// cutlass::layout::{RowMajor,ColumnMajor}, cutlass::TensorRef); this library
// does not depend on CUTLASS and defines the small subset the SRGEMM operators
// use (include/cuasr/gemm/device/srgemm.h:139-183 of the reference).
#pragma once
#include <cstddef>
#include <cstdint>
#include <limits>

#include "../cuasr_amd.h"

namespace cuasr {

/// Same enumerators, same order as cutlass::Status (static_cast<int> agrees
/// with the C ABI's cuasr_amd_status).
enum class Status {
  kSuccess = CUASR_AMD_SUCCESS,
  kErrorMisalignedOperand,
  kErrorInvalidDataType,
  kErrorInvalidLayout,
  kErrorInvalidProblem,
  kErrorNotSupported,
  kErrorWorkspaceNull,
  kErrorInternal,
  kErrorArchMismatch,
  kErrorInsufficientDriver,
  kErrorMemoryAllocation,
  kInvalid
};

inline char const *cuasrGetStatusString(Status s) { return cuasr_amd_status_string(static_cast<int>(s)); }

struct MatrixCoord {
  int r, c;
  MatrixCoord(int row = 0, int column = 0) : r(row), c(column) {}
  int row() const { return r; }
  int column() const { return c; }
};

namespace gemm {

struct GemmCoord {
  int mnk[3];
  GemmCoord(int m = 0, int n = 0, int k = 0) : mnk{m, n, k} {}
  int m() const { return mnk[0]; }
  int n() const { return mnk[1]; }
  int k() const { return mnk[2]; }
  int &m() { return mnk[0]; }
  int &n() { return mnk[1]; }
  int &k() { return mnk[2]; }
};

/// Compile-time tile shape; accepted by the operator templates for source
/// compatibility (tiling is chosen by the library, not by these values).
template <int M, int N, int K> struct GemmShape {
  static int const kM = M, kN = N, kK = K;
};

namespace threadblock {
template <int N = 1> struct GemmIdentityThreadblockSwizzle {};
struct GemmSplitKHorizontalThreadblockSwizzle {};
}  // namespace threadblock
}  // namespace gemm

namespace arch {
struct OpClassSimt {};      ///< the reference's only class; here: the library picks the kernel family
struct OpClassMatrixCore {};///< matrix-core assisted kernels
struct OpClassVectorAlu {}; ///< vector-ALU tiles only: bit-exact sequential sums also for plus-times
struct Gfx950 {};           ///< MI355X
using Sm50 = Gfx950;        ///< spelled by existing cuASR user code; selects the same kernels
}  // namespace arch

namespace layout {
struct ColumnMajor {
  static int const kRank = 2;
  static int const kAbiTag = CUASR_AMD_COLUMN_MAJOR;
  long long ld;
  ColumnMajor(long long ldm = 0) : ld(ldm) {}
  long long operator()(MatrixCoord const &c) const { return c.row() + c.column() * ld; }
  long long stride(int = 0) const { return ld; }
};
struct RowMajor {
  static int const kRank = 2;
  static int const kAbiTag = CUASR_AMD_ROW_MAJOR;
  long long ld;
  RowMajor(long long ldm = 0) : ld(ldm) {}
  long long operator()(MatrixCoord const &c) const { return c.row() * ld + c.column(); }
  long long stride(int = 0) const { return ld; }
};
}  // namespace layout

/// Pointer + layout.  Brace-initialisable from {ptr, ld} like cutlass::TensorRef.
template <typename Element, typename Layout> class TensorRef {
 public:
  TensorRef() : ptr_(nullptr), layout_(0) {}
  TensorRef(Element *ptr, Layout const &layout) : ptr_(ptr), layout_(layout) {}
  TensorRef(Element *ptr, long long ld) : ptr_(ptr), layout_(ld) {}
  /// const-qualifying conversion (TensorRef<T> -> TensorRef<T const>)
  template <typename U, typename = decltype(static_cast<Element *>(static_cast<U *>(nullptr)))>
  TensorRef(TensorRef<U, Layout> const &o) : ptr_(o.data()), layout_(o.layout()) {}
  Element *data() const { return ptr_; }
  Layout const &layout() const { return layout_; }
  long long stride(int = 0) const { return layout_.ld; }
  Element &at(MatrixCoord const &c) const { return ptr_[layout_(c)]; }
  void reset(Element *ptr) { ptr_ = ptr; }

 private:
  Element *ptr_;
  Layout layout_;
};

/// IEEE binary16 for host code that has no such arithmetic type (g++ on x86-64 before version 12): two bytes of
/// storage, every operation carried out in float and rounded back to nearest-even -- float's 24 digits are enough for
/// the sum, product or quotient of two binary16 values to round as if computed exactly.  What the reference would
/// use cutlass::half_t for (it names half precision as an aim only, README.md:11).  Device memory holds the same
/// two bytes; the library's kernels compute on them natively.
struct half_t {
  uint16_t bits;
  constexpr half_t() : bits(0) {}
  template <typename U, typename = decltype(static_cast<float>(U()))> constexpr half_t(U v) : bits(round(static_cast<float>(v))) {}
  constexpr operator float() const { return widen(bits); }
  static constexpr half_t from_bits(uint16_t b) { half_t h; h.bits = b; return h; }

  static constexpr uint16_t round(float f) {
    const uint32_t x = __builtin_bit_cast(uint32_t, f);
    const uint32_t sign = (x >> 16) & 0x8000u, mag = x & 0x7fffffffu;
    if (mag > 0x7f800000u) return static_cast<uint16_t>(sign | 0x7e00u);           // NaN
    if (mag >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);          // rounds to infinity (>= 65520)
    if (mag < 0x33000001u) return static_cast<uint16_t>(sign);                     // <= 2^-25: rounds to zero
    const int e = static_cast<int>(mag >> 23) - 127;                               // unbiased exponent, -25 .. 15
    const uint32_t m = (mag & 0x7fffffu) | 0x800000u;                              // 24 significant bits
    const int drop = e >= -14 ? 13 : 13 + (-14 - e);                               // bits below the binary16 mantissa
    uint32_t kept = m >> drop;
    const uint32_t rest = m & ((1u << drop) - 1u), half = 1u << (drop - 1);
    if (rest > half || (rest == half && (kept & 1u))) ++kept;                      // to nearest, ties to even
    // normal: kept has its leading one at bit 10, which adds 1 to the exponent field; a carry out of the
    // mantissa moves into the exponent by itself (also from the largest subnormal into the smallest normal)
    const uint32_t h = e >= -14 ? (static_cast<uint32_t>(e + 14) << 10) + kept : kept;
    return static_cast<uint16_t>(sign | h);
  }
  static constexpr float widen(uint16_t b) {
    const uint32_t sign = static_cast<uint32_t>(b & 0x8000u) << 16, e = (b >> 10) & 0x1fu, m = b & 0x3ffu;
    if (e == 31) return __builtin_bit_cast(float, sign | 0x7f800000u | (m << 13));
    if (e != 0) return __builtin_bit_cast(float, sign | ((e + 112u) << 23) | (m << 13));
    const float v = static_cast<float>(m) * 5.9604644775390625e-8f;                // subnormal: m * 2^-24, exact
    return sign ? -v : v;
  }
};
static_assert(sizeof(half_t) == 2, "binary16 is two bytes");

}  // namespace cuasr

namespace std {
template <> struct numeric_limits<cuasr::half_t> {
  static constexpr bool is_specialized = true, is_signed = true, is_integer = false, is_exact = false, has_infinity = true,
                        has_quiet_NaN = true;
  static constexpr int digits = 11;
  static constexpr cuasr::half_t min() { return cuasr::half_t::from_bits(0x0400); }       // smallest positive normal
  static constexpr cuasr::half_t max() { return cuasr::half_t::from_bits(0x7bff); }       // 65504
  static constexpr cuasr::half_t lowest() { return cuasr::half_t::from_bits(0xfbff); }
  static constexpr cuasr::half_t infinity() { return cuasr::half_t::from_bits(0x7c00); }
  static constexpr cuasr::half_t quiet_NaN() { return cuasr::half_t::from_bits(0x7e00); }
  static constexpr cuasr::half_t epsilon() { return cuasr::half_t::from_bits(0x1400); }   // 2^-10
};
}  // namespace std

namespace cuasr {

/// element type -> cuasr_amd_dtype
template <typename T> struct dtype_tag;
template <> struct dtype_tag<half_t> { static int const value = CUASR_AMD_F16; };
template <> struct dtype_tag<float> { static int const value = CUASR_AMD_F32; };
template <> struct dtype_tag<double> { static int const value = CUASR_AMD_F64; };
template <> struct dtype_tag<int32_t> { static int const value = CUASR_AMD_I32; };
template <> struct dtype_tag<uint32_t> { static int const value = CUASR_AMD_U32; };

/// (operand type, result type) -> cuasr_amd_dtype: one type throughout, or int8 operands with int32 results
/// (the element types of the reference's dp4a cores, default_srmma_core_simt.h:747-757)
template <typename TA, typename TB, typename TC, typename TAcc> struct element_types {
  static bool const valid = false;
  static int const value = -1;
};
template <typename T> struct element_types<T, T, T, T> {
  static bool const valid = true;
  static int const value = dtype_tag<T>::value;
};
template <> struct element_types<int8_t, int8_t, int32_t, int32_t> {
  static bool const valid = true;
  static int const value = CUASR_AMD_I8;
};
/// binary16 operands and results with a float accumulator: plus-times on the matrix cores, sums in float, D rounded
/// to binary16 once (the library runs this only when asked to: device::Srgemm asks by this accumulator type)
template <> struct element_types<half_t, half_t, half_t, float> {
  static bool const valid = true;
  static int const value = CUASR_AMD_F16;
};

template <typename T> inline cuasr_amd_scalar make_scalar(T v);
template <> inline cuasr_amd_scalar make_scalar<half_t>(half_t v) { cuasr_amd_scalar s; s.bits = 0; s.f16 = v.bits; return s; }
template <> inline cuasr_amd_scalar make_scalar<float>(float v) { cuasr_amd_scalar s; s.bits = 0; s.f32 = v; return s; }
template <> inline cuasr_amd_scalar make_scalar<double>(double v) { cuasr_amd_scalar s; s.bits = 0; s.f64 = v; return s; }
template <> inline cuasr_amd_scalar make_scalar<int32_t>(int32_t v) { cuasr_amd_scalar s; s.bits = 0; s.i32 = v; return s; }
template <> inline cuasr_amd_scalar make_scalar<uint32_t>(uint32_t v) { cuasr_amd_scalar s; s.bits = 0; s.u32 = v; return s; }

}  // namespace cuasr

#if !defined(CUASR_AMD_NO_CUTLASS_NAMES) && !defined(CUTLASS_HOST_DEVICE)
#include "cutlass_names.h"
#endif
