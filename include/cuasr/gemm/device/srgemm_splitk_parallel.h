// cuasr::gemm::device::SrgemmSplitKParallel -- two-kernel parallel split-K:
// partial products of `split_k_slices` K-slices go to a caller-provided
// workspace, a second kernel folds them with the semiring's add and applies
// the epilogue.  Mirrors include/cuasr/gemm/device/srgemm_splitk_parallel.h
// :36-378 (and :424-607) of the reference: same template head, Arguments,
// get_workspace_size = sizeof(accumulator) * M * N * slices, initialize(args,
// workspace) returning kErrorWorkspaceNull for a null workspace, run(stream).
#pragma once
#include "srgemm.h"

namespace cuasr {
namespace reduction {
namespace thread {
/// Named by the reference's template head; carries no state here.
template <typename AdditionOp, typename ElementAccumulator, typename Element, int Count = 1> struct SemiringReduce {
  struct Params {};
};
}  // namespace thread
}  // namespace reduction
namespace epilogue {
namespace thread {
template <typename Element, int Count = 1, typename ElementOut = Element> struct Convert {
  struct Params {};
};
}  // namespace thread
}  // namespace epilogue

namespace gemm {
namespace device {

template <typename AdditionOp_, typename MultiplicationOp_, typename ElementA_, typename LayoutA_, typename ElementB_,
          typename LayoutB_, typename ElementC_, typename LayoutC_, typename ElementAccumulator_ = ElementC_,
          typename OperatorClass_ = arch::OpClassSimt, typename ArchTag_ = arch::Gfx950,
          typename ThreadblockShape_ = typename DefaultSemiRingConfiguration<
              ElementA_, ElementB_, ElementC_, ElementAccumulator_, OperatorClass_, AdditionOp_, MultiplicationOp_,
              ArchTag_>::ThreadblockShape,
          typename WarpShape_ = typename DefaultSemiRingConfiguration<ElementA_, ElementB_, ElementC_, ElementAccumulator_,
                                                                     OperatorClass_, AdditionOp_, MultiplicationOp_,
                                                                     ArchTag_>::WarpShape,
          typename InstructionShape_ = typename DefaultSemiRingConfiguration<
              ElementA_, ElementB_, ElementC_, ElementAccumulator_, OperatorClass_, AdditionOp_, MultiplicationOp_,
              ArchTag_>::InstructionShape,
          typename EpilogueOutputOp_ = typename DefaultSemiRingConfiguration<
              ElementA_, ElementB_, ElementC_, ElementAccumulator_, OperatorClass_, AdditionOp_, MultiplicationOp_,
              ArchTag_>::EpilogueOutputOp,
          typename ConvertScaledOp_ = epilogue::thread::Convert<ElementAccumulator_, 1, ElementAccumulator_>,
          typename ReductionOp_ = reduction::thread::SemiringReduce<AdditionOp_, ElementAccumulator_, ElementAccumulator_, 1>,
          typename ThreadblockSwizzle_ = threadblock::GemmSplitKHorizontalThreadblockSwizzle,
          int Stages = DefaultSemiRingConfiguration<ElementA_, ElementB_, ElementC_, ElementAccumulator_, OperatorClass_,
                                                    AdditionOp_, MultiplicationOp_, ArchTag_>::kStages,
          int kAlignmentA = 1, int kAlignmentB = 1>
class SrgemmSplitKParallel {
 public:
  using ElementA = ElementA_;
  using LayoutA = LayoutA_;
  using ElementB = ElementB_;
  using LayoutB = LayoutB_;
  using ElementC = ElementC_;
  using LayoutC = LayoutC_;
  using ElementAccumulator = ElementAccumulator_;
  using OperatorClass = OperatorClass_;
  using ArchTag = ArchTag_;
  using ThreadblockShape = ThreadblockShape_;
  using WarpShape = WarpShape_;
  using InstructionShape = InstructionShape_;
  using EpilogueOutputOp = EpilogueOutputOp_;
  using ConvertScaledOp = ConvertScaledOp_;
  using ReductionOp = ReductionOp_;
  using ThreadblockSwizzle = ThreadblockSwizzle_;
  using AdditionOp = AdditionOp_;
  using MultiplicationOp = MultiplicationOp_;
  static int const kStages = Stages;
  /// true when AdditionOp or MultiplicationOp is none of the library's operators: the slice kernel and the
  /// reduction are then built from the functors' operator() in this translation unit
  /// (cuasr/gemm/kernel/functor_srgemm.h, cuasr/reduction/kernel/reduce_split_k.h), which needs hipcc
  static bool const kUserFunctors = op_tag<AdditionOp>::value < 0 || op_tag<MultiplicationOp>::value < 0;
  static_assert(!kUserFunctors || (std::is_same<ElementA, ElementC>::value && sizeof(ElementC) >= 4),
                "kernels built from user functors: float, double, int32_t or uint32_t throughout");

  static_assert(element_types<ElementA, ElementB, ElementC, ElementAccumulator>::valid,
                "A, B, C and the accumulator share one element type (as in every reference configuration), or A and B "
                "are int8_t with int32_t C and accumulator, or all three are half_t with a float accumulator (plus-times "
                "only: every other pair computes in binary16 throughout and is refused by can_implement with that "
                "accumulator -- name half_t as the accumulator type instead)");

  struct Arguments {
    GemmCoord problem_size;
    TensorRef<ElementA const, LayoutA> ref_A;
    TensorRef<ElementB const, LayoutB> ref_B;
    TensorRef<ElementC const, LayoutC> ref_C;
    TensorRef<ElementC, LayoutC> ref_D;
    typename EpilogueOutputOp::Params epilogue;
    int split_k_slices;
    typename ConvertScaledOp::Params convert;
    typename ReductionOp::Params reduction;

    Arguments() : problem_size(0, 0, 0), split_k_slices(1) {}
    Arguments(GemmCoord problem_size_, TensorRef<ElementA const, LayoutA> ref_A_, TensorRef<ElementB const, LayoutB> ref_B_,
              TensorRef<ElementC const, LayoutC> ref_C_, TensorRef<ElementC, LayoutC> ref_D_,
              typename EpilogueOutputOp::Params epilogue_ = typename EpilogueOutputOp::Params(), int split_k_slices_ = 1,
              typename ConvertScaledOp::Params convert_ = typename ConvertScaledOp::Params(),
              typename ReductionOp::Params reduction_ = typename ReductionOp::Params())
        : problem_size(problem_size_), ref_A(ref_A_), ref_B(ref_B_), ref_C(ref_C_), ref_D(ref_D_), epilogue(epilogue_),
          split_k_slices(split_k_slices_), convert(convert_), reduction(reduction_) {}
  };

  SrgemmSplitKParallel() : workspace_(nullptr), ready_(false) {}

  /// Stricter than the reference's stub (which always succeeds): the
  /// descriptor is validated, slices must be >= 1.
  static Status can_implement(Arguments const &args) {
    if (args.split_k_slices < 1) return Status::kErrorInvalidProblem;
    if constexpr (kUserFunctors) return detail::functor_check<SrgemmSplitKParallel>(args);
    Arguments one = args;
    one.split_k_slices = 1;
    cuasr_amd_srgemm_desc d = detail::make_desc<SrgemmSplitKParallel>(one, detail::kernel_of<OperatorClass>::value);
    return static_cast<Status>(cuasr_amd_srgemm_can_implement(&d));
  }

  static size_t get_workspace_size(Arguments const &args) {
    if constexpr (kUserFunctors) {
      if (args.problem_size.m() < 0 || args.problem_size.n() < 0 || args.split_k_slices < 1) return 0;
      return sizeof(ElementAccumulator) * size_t(args.problem_size.m()) * size_t(args.problem_size.n()) * size_t(args.split_k_slices);
    }
    cuasr_amd_srgemm_desc d = detail::make_desc<SrgemmSplitKParallel>(args, CUASR_AMD_KERNEL_AUTO);
    return cuasr_amd_splitk_workspace_bytes(&d);
  }

  Status initialize(Arguments const &args, void *workspace) {
    if (!workspace) return Status::kErrorWorkspaceNull;
    Status s = can_implement(args);
    if (s != Status::kSuccess) return s;
    args_ = args;
    if constexpr (!kUserFunctors) desc_ = detail::make_desc<SrgemmSplitKParallel>(args, detail::kernel_of<OperatorClass>::value);
    workspace_ = workspace;
    ready_ = true;
    return Status::kSuccess;
  }

  Status update(Arguments const &args, void *workspace = nullptr) {
    if (!workspace) return Status::kErrorWorkspaceNull;
    if (!ready_) return Status::kErrorInternal;
    args_.ref_A = args.ref_A;
    args_.ref_B = args.ref_B;
    args_.ref_C = args.ref_C;
    args_.ref_D = args.ref_D;
    desc_.A = args.ref_A.data();
    desc_.B = args.ref_B.data();
    desc_.C = args.ref_C.data();
    desc_.D = args.ref_D.data();
    workspace_ = workspace;
    return Status::kSuccess;
  }

  Status run(hipStream_t stream = nullptr) {
    if (!ready_) return Status::kErrorInternal;
    if constexpr (kUserFunctors) {
#if defined(__HIPCC__)
      return detail::functor_splitk<SrgemmSplitKParallel>(args_, workspace_, false, stream);
#else
      static_assert(!kUserFunctors,
                    "cuasr::gemm::device::SrgemmSplitKParallel: AdditionOp / MultiplicationOp is not one of the library's "
                    "operators (no cuasr::op_tag specialisation), so its kernels have to be built from the functors: "
                    "compile this translation unit with hipcc, or specialise cuasr::op_tag if the functor is one of them");
      return Status::kErrorNotSupported;
#endif
    }
    return static_cast<Status>(cuasr_amd_srgemm_splitk(&desc_, workspace_, stream));
  }

  Status operator()(hipStream_t stream = nullptr) { return run(stream); }

  Status operator()(Arguments const &args, void *workspace = nullptr, hipStream_t stream = nullptr) {
    Status s = initialize(args, workspace);
    return s == Status::kSuccess ? run(stream) : s;
  }

 private:
  Arguments args_;
  cuasr_amd_srgemm_desc desc_;
  void *workspace_;
  bool ready_;
};

}  // namespace device
}  // namespace gemm
}  // namespace cuasr
