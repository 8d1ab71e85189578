// Per-semiring default configuration of the cuASR API
// (include/cuasr/gemm/device/default_srgemm_configuration.h:44-275 of the
// reference).  The reference uses it to pick CUDA tile shapes; here the shapes
// are descriptive only -- they state the tile the gfx950 kernels use for that
// element size -- and the type mainly supplies EpilogueOutputOp.
#pragma once
#include "../epilogue/thread/semiring_linear_combination.h"

namespace cuasr {
namespace gemm {
namespace device {

template <typename ElementA, typename ElementB, typename ElementC, typename ElementAccumulator, typename OperatorClass,
          typename AdditionOp, typename MultiplicationOp, typename ArchTag>
struct DefaultSemiRingConfiguration {
  static int const kAlignmentA = 1;
  static int const kAlignmentB = 1;
  /// workgroup tile of the vector-ALU kernels: 128 x 128 x 16 for 4-byte
  /// elements, 128 x 64 x 8 for 8-byte elements; one wave64 owns a 32 x 128
  /// (resp. 32 x 64) strip of it
  using ThreadblockShape = GemmShape<128, (sizeof(ElementC) == 8 ? 64 : 128), (sizeof(ElementC) == 8 ? 8 : 16)>;
  using WarpShape = GemmShape<32, (sizeof(ElementC) == 8 ? 64 : 128), (sizeof(ElementC) == 8 ? 8 : 16)>;
  using InstructionShape = GemmShape<1, 1, 1>;
  static int const kStages = 2;
  using EpilogueOutputOp =
      epilogue::thread::SemiringLinearCombination<AdditionOp, MultiplicationOp, ElementC, 1, ElementAccumulator, ElementAccumulator>;
};

}  // namespace device
}  // namespace gemm
}  // namespace cuasr
