// Matrix-core assisted kernels for float (placeholder table until the tile lands).
#include "semiring.h"

namespace cuasr_amd {

launch_fn find_mfma_f32(int, int) { return nullptr; }

}  // namespace cuasr_amd
