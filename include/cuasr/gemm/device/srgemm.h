// cuasr::gemm::device::Srgemm -- the cuASR device-level SRGEMM operator,
// implemented on libcuasr_amd (hand-written gfx950 kernels behind a C ABI).
//
// Same template head, member aliases, Arguments and methods as the reference
// operator (include/cuasr/gemm/device/srgemm.h:28-357 and the column-major
// specialisation :398-567); `cudaStream_t` becomes `hipStream_t`.  The tile
// shape / swizzle / stage parameters are accepted and ignored: tiling is the
// library's business.  Column-major C needs no specialisation here -- the
// library runs the transposed problem itself.
//
// Ownership and threading follow the reference: the caller owns A, B, C, D and
// the workspace (device memory); the operator object holds a by-value copy of
// the arguments; nothing allocates or synchronises; launches are asynchronous
// on the given stream; D may alias C.
#pragma once
#include <hip/hip_runtime_api.h>

#include <type_traits>

#include "default_srgemm_configuration.h"
#if defined(__HIPCC__)
#include "../../reduction/kernel/reduce_split_k.h"
#include "../kernel/functor_srgemm.h"
#endif

namespace cuasr {
namespace gemm {
namespace device {

namespace detail {
/// Fill the C-ABI descriptor from typed arguments.
template <typename Op, typename Args>
inline cuasr_amd_srgemm_desc make_desc(Args const &a, int kernel) {
  using Element = typename Op::ElementC;
  cuasr_amd_srgemm_desc d{};
  d.add_op = op_tag<typename Op::AdditionOp>::value;
  d.mult_op = op_tag<typename Op::MultiplicationOp>::value;
  d.dtype = element_types<typename Op::ElementA, typename Op::ElementB, Element, typename Op::ElementAccumulator>::value;
  d.layout_a = Op::LayoutA::kAbiTag;
  d.layout_b = Op::LayoutB::kAbiTag;
  d.layout_c = Op::LayoutC::kAbiTag;
  d.m = a.problem_size.m();
  d.n = a.problem_size.n();
  d.k = a.problem_size.k();
  d.split_k_slices = a.split_k_slices;
  d.A = a.ref_A.data(); d.lda = a.ref_A.stride(0);
  d.B = a.ref_B.data(); d.ldb = a.ref_B.stride(0);
  d.C = a.ref_C.data(); d.ldc = a.ref_C.stride(0);
  d.D = a.ref_D.data(); d.ldd = a.ref_D.stride(0);
  d.alpha = make_scalar<Element>(a.epilogue.alpha);
  d.beta = make_scalar<Element>(a.epilogue.beta);
  d.add_identity = make_scalar<Element>(Op::AdditionOp::Identity);
  d.mult_identity = make_scalar<Element>(Op::MultiplicationOp::Identity);
  d.alpha_ptr = a.epilogue.alpha_ptr;
  d.beta_ptr = a.epilogue.beta_ptr;
  d.kernel = kernel;
  // half operands with a float accumulator (plus-times only, see the operator's static_assert): the matrix-core
  // kernel is the one that accumulates in float
  if (std::is_same<typename Op::ElementC, half_t>::value && std::is_same<typename Op::ElementAccumulator, float>::value)
    d.kernel = CUASR_AMD_KERNEL_MFMA;
  d.reserved = 0;
  return d;
}
/// k-tile depth the reference's default configurations slice K by (ThreadblockShape::kK = 8 in every one of
/// them, device/default_srgemm_configuration.h:44-275); kernels built from user functors follow its slice
/// rules with this depth, because their results may depend on where a slice ends.
static int const kReferenceTileK = 8;

/// The host-side checks of a problem that runs on kernels built from user functors (no C-ABI descriptor to validate).
template <typename Op, typename Args> inline Status functor_check(Args const &args) {
  const long long m = args.problem_size.m(), n = args.problem_size.n(), k = args.problem_size.k();
  if (m < 0 || n < 0 || k < 0 || args.split_k_slices < 1 || args.split_k_slices > 65535) return Status::kErrorInvalidProblem;
  auto ld_ok = [](long long ld, bool column_major, long long rows, long long cols) { return ld >= (column_major ? rows : cols); };
  if (m > 0 && k > 0 && !ld_ok(args.ref_A.stride(0), Op::LayoutA::kAbiTag == CUASR_AMD_COLUMN_MAJOR, m, k)) return Status::kErrorInvalidProblem;
  if (n > 0 && k > 0 && !ld_ok(args.ref_B.stride(0), Op::LayoutB::kAbiTag == CUASR_AMD_COLUMN_MAJOR, k, n)) return Status::kErrorInvalidProblem;
  if (m > 0 && n > 0) {
    if (!args.ref_D.data() || !ld_ok(args.ref_D.stride(0), Op::LayoutC::kAbiTag == CUASR_AMD_COLUMN_MAJOR, m, n)) return Status::kErrorInvalidProblem;
    if (args.ref_C.data() && !ld_ok(args.ref_C.stride(0), Op::LayoutC::kAbiTag == CUASR_AMD_COLUMN_MAJOR, m, n)) return Status::kErrorInvalidProblem;
    if (k > 0 && (!args.ref_A.data() || !args.ref_B.data())) return Status::kErrorInvalidProblem;
  }
  return Status::kSuccess;
}

#if defined(__HIPCC__)
/// Typed arguments -> the parameters of the functor kernel (one slice, epilogue in the kernel).
template <typename Op, typename Args> inline kernel::FunctorSrgemmParams<typename Op::ElementC> functor_params(Args const &a) {
  using Element = typename Op::ElementC;
  kernel::FunctorSrgemmParams<Element> p{};
  p.m = a.problem_size.m();
  p.n = a.problem_size.n();
  p.k = a.problem_size.k();
  auto strides = [](long long ld, bool column_major, long long &s_row, long long &s_col) {
    s_row = column_major ? 1 : ld;
    s_col = column_major ? ld : 1;
  };
  p.A = a.ref_A.data();
  strides(a.ref_A.stride(0), Op::LayoutA::kAbiTag == CUASR_AMD_COLUMN_MAJOR, p.sa_m, p.sa_k);
  p.B = a.ref_B.data();
  strides(a.ref_B.stride(0), Op::LayoutB::kAbiTag == CUASR_AMD_COLUMN_MAJOR, p.sb_k, p.sb_n);
  p.C = a.ref_C.data();
  strides(a.ref_C.stride(0), Op::LayoutC::kAbiTag == CUASR_AMD_COLUMN_MAJOR, p.sc_m, p.sc_n);
  p.D = a.ref_D.data();
  strides(a.ref_D.stride(0), Op::LayoutC::kAbiTag == CUASR_AMD_COLUMN_MAJOR, p.sd_m, p.sd_n);
  p.alpha = a.epilogue.alpha;
  p.beta = a.epilogue.beta;
  p.alpha_ptr = static_cast<Element const *>(a.epilogue.alpha_ptr);
  p.beta_ptr = static_cast<Element const *>(a.epilogue.beta_ptr);
  p.workspace = nullptr;
  p.slices = 1;
  p.k_per_slice = p.k;
  p.last_takes_rest = 0;
  return p;
}

/// Both split-K forms on kernels built from the functors: the slices' raw accumulators into the workspace
/// (one launch, the slice index in the grid), then the fold + epilogue.  k_per_slice follows the reference:
/// parallel ((K / 8) / S) * 8 with the last slice running on to K (kernel/srgemm_splitk_parallel.h:86-89,
/// :136-142), serial ceil(ceil(K / 8) / S) * 8 with every slice cut off at K (kernel/srgemm.h:97-100, :184-189).
template <typename Op, typename Args> inline Status functor_splitk(Args const &a, void *workspace, bool serial, hipStream_t stream) {
  using Element = typename Op::ElementC;
  using Add = typename Op::AdditionOp;
  using Mult = typename Op::MultiplicationOp;
  kernel::FunctorSrgemmParams<Element> p = functor_params<Op>(a);
  const int slices = a.split_k_slices;
  p.workspace = static_cast<Element *>(workspace);
  p.slices = slices;
  const long long tk = kReferenceTileK;
  if (serial) {
    const long long iterations = (p.k + tk - 1) / tk;
    p.k_per_slice = (int)(((iterations + slices - 1) / slices) * tk);
    p.last_takes_rest = 0;
  } else {
    p.k_per_slice = (int)(((p.k / tk) / slices) * tk);
    p.last_takes_rest = 1;
  }
  if (kernel::launch_functor_srgemm<Add, Mult, Element>(p, stream) != hipSuccess) return Status::kErrorInternal;
  reduction::kernel::FunctorReduceParams<Element> r{};
  r.m = p.m; r.n = p.n; r.slices = slices;
  r.workspace = p.workspace;
  r.C = p.C; r.sc_m = p.sc_m; r.sc_n = p.sc_n;
  r.D = p.D; r.sd_m = p.sd_m; r.sd_n = p.sd_n;
  r.alpha = p.alpha; r.beta = p.beta; r.alpha_ptr = p.alpha_ptr; r.beta_ptr = p.beta_ptr;
  return reduction::kernel::launch_functor_reduce<Add, Mult, Element>(r, serial, stream) == hipSuccess ? Status::kSuccess
                                                                                                      : Status::kErrorInternal;
}
#endif

template <typename OperatorClass> struct kernel_of { static int const value = CUASR_AMD_KERNEL_AUTO; };
template <> struct kernel_of<arch::OpClassMatrixCore> { static int const value = CUASR_AMD_KERNEL_MFMA; };
template <> struct kernel_of<arch::OpClassVectorAlu> { static int const value = CUASR_AMD_KERNEL_VALU; };
}  // namespace detail

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
          typename ThreadblockSwizzle_ = threadblock::GemmIdentityThreadblockSwizzle<>,
          int Stages = DefaultSemiRingConfiguration<ElementA_, ElementB_, ElementC_, ElementAccumulator_, OperatorClass_,
                                                    AdditionOp_, MultiplicationOp_, ArchTag_>::kStages,
          int AlignmentA = DefaultSemiRingConfiguration<ElementA_, ElementB_, ElementC_, ElementAccumulator_, OperatorClass_,
                                                        AdditionOp_, MultiplicationOp_, ArchTag_>::kAlignmentA,
          int AlignmentB = DefaultSemiRingConfiguration<ElementA_, ElementB_, ElementC_, ElementAccumulator_, OperatorClass_,
                                                        AdditionOp_, MultiplicationOp_, ArchTag_>::kAlignmentB,
          bool SplitKSerial = false>
class Srgemm {
 public:
  using ElementA = ElementA_;
  using LayoutA = LayoutA_;
  using TensorRefA = TensorRef<ElementA const, LayoutA>;
  using ElementB = ElementB_;
  using LayoutB = LayoutB_;
  using TensorRefB = TensorRef<ElementB const, LayoutB>;
  using ElementC = ElementC_;
  using LayoutC = LayoutC_;
  using TensorRefC = TensorRef<ElementC const, LayoutC>;
  using TensorRefD = TensorRef<ElementC, LayoutC>;
  using ElementAccumulator = ElementAccumulator_;
  using OperatorClass = OperatorClass_;
  using ArchTag = ArchTag_;
  using ThreadblockShape = ThreadblockShape_;
  using WarpShape = WarpShape_;
  using InstructionShape = InstructionShape_;
  using EpilogueOutputOp = EpilogueOutputOp_;
  using ThreadblockSwizzle = ThreadblockSwizzle_;
  using AdditionOp = AdditionOp_;
  using MultiplicationOp = MultiplicationOp_;
  static int const kStages = Stages;
  static int const kAlignmentA = AlignmentA;
  static int const kAlignmentB = AlignmentB;
  static int const kAlignmentC = EpilogueOutputOp::kCount;
  static bool const kSplitKSerial = SplitKSerial;
  /// true when AdditionOp or MultiplicationOp is none of the library's operators (no cuasr::op_tag
  /// specialisation): the kernel is then built from the functors' operator() in this translation unit
  /// (cuasr/gemm/kernel/functor_srgemm.h), which needs hipcc; the serial split-K runs on the same kernel plus the
  /// replay of the slices' epilogues in cuasr/reduction/kernel/reduce_split_k.h
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

    Arguments() : problem_size(0, 0, 0), split_k_slices(1) {}
    Arguments(GemmCoord problem_size_, TensorRef<ElementA const, LayoutA> ref_A_, TensorRef<ElementB const, LayoutB> ref_B_,
              TensorRef<ElementC const, LayoutC> ref_C_, TensorRef<ElementC, LayoutC> ref_D_,
              typename EpilogueOutputOp::Params epilogue_ = typename EpilogueOutputOp::Params(), int split_k_slices_ = 1)
        : problem_size(problem_size_), ref_A(ref_A_), ref_B(ref_B_), ref_C(ref_C_), ref_D(ref_D_), epilogue(epilogue_),
          split_k_slices(split_k_slices_) {}
  };

  Srgemm() : workspace_(nullptr), ready_(false) {}

  /// kErrorInvalidProblem when split_k_slices > 1 and SplitKSerial is false
  /// (reference: srgemm.h:198-200).
  static Status can_implement(Arguments const &args) {
    if (!kSplitKSerial && args.split_k_slices > 1) return Status::kErrorInvalidProblem;
    if (args.split_k_slices < 1) return Status::kErrorInvalidProblem;
    if constexpr (kUserFunctors) return detail::functor_check<Srgemm>(args);
    cuasr_amd_srgemm_desc d = detail::make_desc<Srgemm>(args, detail::kernel_of<OperatorClass>::value);
    d.split_k_slices = 1;  // the slice count is checked above; the rest is the plain problem's check
    return static_cast<Status>(cuasr_amd_srgemm_can_implement(&d));
  }

  /// Serial split-K: bytes of device workspace `initialize` must be given
  /// (reference: srgemm.h:218-234).  The reference needs one int per output tile
  /// for its semaphores; this library needs the slices' partial products,
  /// sizeof(ElementC) * M * N * split_k_slices, so size the workspace with this
  /// function, as the reference's callers do.
  static size_t get_workspace_size(Arguments const &args) {
    if (!kSplitKSerial || args.split_k_slices <= 1) return 0;
    if constexpr (kUserFunctors)
      return sizeof(ElementC) * size_t(args.problem_size.m()) * size_t(args.problem_size.n()) * size_t(args.split_k_slices);
    cuasr_amd_srgemm_desc d = detail::make_desc<Srgemm>(args, detail::kernel_of<OperatorClass>::value);
    return cuasr_amd_splitk_serial_workspace_bytes(&d);
  }

  /// kErrorWorkspaceNull for a serial split-K without workspace (reference:
  /// srgemm.h:246-251).  Nothing is cleared: the workspace carries no state
  /// from one run to the next.
  Status initialize(Arguments const &args, void *workspace = nullptr, hipStream_t /*stream*/ = nullptr) {
    Status s = can_implement(args);
    if (s != Status::kSuccess) return s;
    if (kSplitKSerial && args.split_k_slices > 1 && !workspace) return Status::kErrorWorkspaceNull;
    args_ = args;
    if constexpr (!kUserFunctors) desc_ = detail::make_desc<Srgemm>(args, detail::kernel_of<OperatorClass>::value);
    workspace_ = workspace;
    ready_ = true;
    return Status::kSuccess;
  }

  /// Lightweight refresh of the operand pointers (reference: srgemm.h:285-300).
  Status update(Arguments const &args, void *workspace = nullptr) {
    if (!ready_) return Status::kErrorInternal;
    if (kSplitKSerial && args.split_k_slices > 1 && !workspace) return Status::kErrorWorkspaceNull;
    args_.ref_A = args.ref_A;
    args_.ref_B = args.ref_B;
    args_.ref_C = args.ref_C;
    args_.ref_D = args.ref_D;
    args_.epilogue = args.epilogue;
    desc_.A = args.ref_A.data();
    desc_.B = args.ref_B.data();
    desc_.C = args.ref_C.data();
    desc_.D = args.ref_D.data();
    desc_.alpha = make_scalar<ElementC>(args.epilogue.alpha);
    desc_.beta = make_scalar<ElementC>(args.epilogue.beta);
    desc_.alpha_ptr = args.epilogue.alpha_ptr;
    desc_.beta_ptr = args.epilogue.beta_ptr;
    workspace_ = workspace;
    return Status::kSuccess;
  }

  Status run(hipStream_t stream = nullptr) {
    if (!ready_) return Status::kErrorInternal;
    if constexpr (kUserFunctors) {
#if defined(__HIPCC__)
      if (kSplitKSerial && args_.split_k_slices > 1) return detail::functor_splitk<Srgemm>(args_, workspace_, true, stream);
      const kernel::FunctorSrgemmParams<ElementC> p = detail::functor_params<Srgemm>(args_);
      return kernel::launch_functor_srgemm<AdditionOp, MultiplicationOp, ElementC>(p, stream) == hipSuccess ? Status::kSuccess
                                                                                                           : Status::kErrorInternal;
#else
      static_assert(!kUserFunctors,
                    "cuasr::gemm::device::Srgemm: AdditionOp / MultiplicationOp is not one of the library's operators "
                    "(plus, multiplies, minimum, maximum, binary_and, binary_or, binary_xor, bitwise_and, bitwise_or; "
                    "no cuasr::op_tag specialisation), so the kernel has to be built from the functor itself: compile "
                    "this translation unit with hipcc, or specialise cuasr::op_tag for the functor if it is one of them");
      return Status::kErrorNotSupported;
#endif
    }
    if (kSplitKSerial && desc_.split_k_slices > 1)
      return static_cast<Status>(cuasr_amd_srgemm_splitk_serial(&desc_, workspace_, stream));
    return static_cast<Status>(cuasr_amd_srgemm(&desc_, stream));
  }

  Status operator()(hipStream_t stream = nullptr) { return run(stream); }

  Status operator()(Arguments const &args, void *workspace = nullptr, hipStream_t stream = nullptr) {
    Status s = initialize(args, workspace, stream);
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
