// The CUTLASS spellings that cuASR user code writes at its call sites, as aliases of this library's own
// types -- names only: no CUTLASS code, no CUDA runtime types.  Reference call sites spell
// cutlass::layout::ColumnMajor / RowMajor, cutlass::arch::OpClassSimt, cutlass::arch::Sm50,
// cutlass::gemm::GemmShape, cutlass::gemm::GemmCoord, cutlass::gemm::threadblock::GemmIdentityThreadblockSwizzle,
// cutlass::Status and cutlass::Array (examples/00_minplus_srgemm/minplus_srgemm.cu:22-35, :61,
// examples/01_userdefined_semiring/userdefined_semiring.cu:68-98, :114-127,
// examples/02_splitk_srgemm/splitk_srgemm.cu:32-42, :74-80; include/cuasr/gemm/device/srgemm.h:139-183 of the
// reference); with this header those lines compile as they are, and only the stream type (hipStream_t) and the
// memory calls of the surrounding program are HIP's.
//
// cuasr/types.h includes this header unless CUASR_AMD_NO_CUTLASS_NAMES is defined or CUTLASS itself is already
// in the translation unit (it defines CUTLASS_HOST_DEVICE), so that a program which has the real CUTLASS keeps it.
#pragma once
#include <hip/hip_runtime_api.h>

#include "array.h"
#include "types.h"

namespace cutlass {

using cuasr::Array;
using cuasr::half_t;
using cuasr::MatrixCoord;
using cuasr::Status;
using cuasr::TensorRef;

inline char const *cutlassGetStatusString(Status s) { return cuasr::cuasrGetStatusString(s); }

namespace layout {
using cuasr::layout::ColumnMajor;
using cuasr::layout::RowMajor;
}  // namespace layout

namespace arch {
using cuasr::arch::OpClassSimt;
// every NVIDIA architecture tag a cuASR program may name selects the one target this library has
using Sm50 = cuasr::arch::Gfx950;
using Sm60 = cuasr::arch::Gfx950;
using Sm61 = cuasr::arch::Gfx950;
using Sm70 = cuasr::arch::Gfx950;
using Sm75 = cuasr::arch::Gfx950;
using Sm80 = cuasr::arch::Gfx950;
}  // namespace arch

namespace gemm {
using cuasr::gemm::GemmCoord;
using cuasr::gemm::GemmShape;
namespace threadblock {
using cuasr::gemm::threadblock::GemmIdentityThreadblockSwizzle;
using cuasr::gemm::threadblock::GemmSplitKHorizontalThreadblockSwizzle;
}  // namespace threadblock
}  // namespace gemm

namespace device_memory {
/// Owning device buffer of `capacity` elements, as the reference's split-K example holds its workspace
/// (examples/02_splitk_srgemm/splitk_srgemm.cu:74-80): allocated on construction, freed on destruction,
/// get() is the device pointer (null for an empty buffer or a failed allocation).
template <typename T> class allocation {
 public:
  allocation() : ptr_(nullptr), capacity_(0) {}
  explicit allocation(size_t capacity) : ptr_(nullptr), capacity_(capacity) {
    if (capacity && hipMalloc(reinterpret_cast<void **>(&ptr_), capacity * sizeof(T)) != hipSuccess) {
      ptr_ = nullptr;
      capacity_ = 0;
    }
  }
  allocation(allocation const &) = delete;
  allocation &operator=(allocation const &) = delete;
  allocation(allocation &&o) noexcept : ptr_(o.ptr_), capacity_(o.capacity_) { o.ptr_ = nullptr; o.capacity_ = 0; }
  allocation &operator=(allocation &&o) noexcept {
    if (this != &o) {
      reset();
      ptr_ = o.ptr_;
      capacity_ = o.capacity_;
      o.ptr_ = nullptr;
      o.capacity_ = 0;
    }
    return *this;
  }
  ~allocation() { reset(); }
  T *get() const { return ptr_; }
  size_t size() const { return capacity_; }
  size_t bytes() const { return capacity_ * sizeof(T); }
  void reset() {
    if (ptr_) (void)hipFree(ptr_);
    ptr_ = nullptr;
    capacity_ = 0;
  }

 private:
  T *ptr_;
  size_t capacity_;
};
}  // namespace device_memory

}  // namespace cutlass
