// Per-semiring default configuration of the cuASR API
// (include/cuasr/gemm/device/default_srgemm_configuration.h:44-275 of the
// reference).  The reference uses it to pick CUDA tile shapes; here the kernel
// (and with it the tile) is chosen at run time by the library, so the shapes
// state the tile of the kernel that serves large aligned problems of that
// element size on gfx950, and the type mainly supplies EpilogueOutputOp and
// the operand alignments device::Srgemm takes its defaults from.
#pragma once
#include "../epilogue/thread/semiring_linear_combination.h"

namespace cuasr {
namespace gemm {
namespace device {

template <typename ElementA, typename ElementB, typename ElementC, typename ElementAccumulator, typename OperatorClass,
          typename AdditionOp, typename MultiplicationOp, typename ArchTag>
struct DefaultSemiRingConfiguration {
  /// in elements, as in the reference (:52-53): every alignment from one element up is served
  static int const kAlignmentA = 1;
  static int const kAlignmentB = 1;
  /// workgroup tile of the direct-to-LDS vector-ALU kernels: 256 x 128 x 16 for 4-byte elements (512 threads,
  /// 8 wave64 of 32 x 128), 128 x 128 x 16 for 8-byte elements (512 threads, 8 wave64 of 16 x 128); a thread
  /// owns 8 x 8 (8 x 4) outputs.  Unaligned, small or oddly sized problems run on 128 x 128 / 64 x 64 tiles.
  using ThreadblockShape = GemmShape<(sizeof(ElementC) == 8 ? 128 : 256), 128, 16>;
  using WarpShape = GemmShape<(sizeof(ElementC) == 8 ? 16 : 32), 128, 16>;
  using InstructionShape = GemmShape<1, 1, 1>;
  /// LDS stages of that kernel
  static int const kStages = sizeof(ElementC) == 8 ? 2 : 3;
  using EpilogueOutputOp =
      epilogue::thread::SemiringLinearCombination<AdditionOp, MultiplicationOp, ElementC, 1, ElementAccumulator, ElementAccumulator>;
};

}  // namespace device
}  // namespace gemm
}  // namespace cuasr
