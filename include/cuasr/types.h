// Value types of the cuASR-compatible operator API: status codes, problem
// coordinates, layouts and tensor references.  The reference takes these from
// CUTLASS (cutlass::Status, cutlass::gemm::GemmCoord, cutlass::MatrixCoord,
// cutlass::layout::{RowMajor,ColumnMajor}, cutlass::TensorRef); this library
// does not depend on CUTLASS and defines the small subset the SRGEMM operators
// use (include/cuasr/gemm/device/srgemm.h:139-183 of the reference).
#pragma once
#include <cstddef>
#include <cstdint>

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

/// element type -> cuasr_amd_dtype
template <typename T> struct dtype_tag;
template <> struct dtype_tag<float> { static int const value = CUASR_AMD_F32; };
template <> struct dtype_tag<double> { static int const value = CUASR_AMD_F64; };
template <> struct dtype_tag<int32_t> { static int const value = CUASR_AMD_I32; };
template <> struct dtype_tag<uint32_t> { static int const value = CUASR_AMD_U32; };

template <typename T> inline cuasr_amd_scalar make_scalar(T v);
template <> inline cuasr_amd_scalar make_scalar<float>(float v) { cuasr_amd_scalar s; s.bits = 0; s.f32 = v; return s; }
template <> inline cuasr_amd_scalar make_scalar<double>(double v) { cuasr_amd_scalar s; s.bits = 0; s.f64 = v; return s; }
template <> inline cuasr_amd_scalar make_scalar<int32_t>(int32_t v) { cuasr_amd_scalar s; s.bits = 0; s.i32 = v; return s; }
template <> inline cuasr_amd_scalar make_scalar<uint32_t>(uint32_t v) { cuasr_amd_scalar s; s.bits = 0; s.u32 = v; return s; }

}  // namespace cuasr
