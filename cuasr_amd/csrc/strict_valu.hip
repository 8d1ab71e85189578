// Vector-ALU tile kernels for the floating-point semirings whose add is a
// comparison and whose mult is `multiplies` (min-times, max-times of
// include/cuasr/gemm/device/default_srgemm_configuration.h:161-218).  Their
// products can be -0, so min/max must keep the reference's comparison
// semantics (functional.h:132, :172) instead of the hardware min/max; this
// file is therefore built WITHOUT the no-NaN assumption the other tile files
// get, which would let the compiler turn the comparisons back into min/max.
#include "valu_tile.h"

namespace cuasr_amd {

launch_fn find_valu_strict(int dtype, int add_op, int mult_op) {
  if (mult_op != kMultiplies) return nullptr;
  if (dtype == CUASR_AMD_F32 && add_op == kMinimum) return launch_valu<float, kMinimum, kMultiplies, 8, 8, 16>;
  if (dtype == CUASR_AMD_F32 && add_op == kMaximum) return launch_valu<float, kMaximum, kMultiplies, 8, 8, 16>;
  if (dtype == CUASR_AMD_F64 && add_op == kMinimum) return launch_valu<double, kMinimum, kMultiplies, 8, 4, 8>;
  if (dtype == CUASR_AMD_F64 && add_op == kMaximum) return launch_valu<double, kMaximum, kMultiplies, 8, 4, 8>;
  return nullptr;
}

}  // namespace cuasr_amd
