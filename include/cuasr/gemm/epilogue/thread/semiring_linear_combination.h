// Epilogue functor of the cuASR API: D = add(mult(alpha, accum), mult(beta, C)).
// Host-side carrier of alpha/beta (by value or by device pointer) with the
// reference's defaults and its is_source_needed rule
// (include/cuasr/gemm/epilogue/thread/semiring_linear_combination.h:54-125 of
// the reference).  The arithmetic itself runs in the device kernels.
#pragma once
#include "../../../functional.h"

namespace cuasr {
namespace epilogue {
namespace thread {

template <typename AdditionOp_, typename MultiplicationOp_, typename ElementOutput_, int Count = 1,
          typename ElementAccumulator_ = ElementOutput_, typename ElementCompute_ = ElementOutput_>
class SemiringLinearCombination {
 public:
  using AdditionOp = AdditionOp_;
  using MultiplicationOp = MultiplicationOp_;
  using ElementOutput = ElementOutput_;
  using ElementAccumulator = ElementAccumulator_;
  using ElementCompute = ElementCompute_;
  static int const kCount = Count;

  struct Params {
    ElementCompute alpha;             ///< scales accumulators
    ElementCompute beta;              ///< scales source tensor
    ElementCompute const *alpha_ptr;  ///< if not null, DEVICE pointer the kernel loads alpha from
    ElementCompute const *beta_ptr;   ///< if not null, DEVICE pointer the kernel loads beta from

    Params() : alpha(MultiplicationOp::Identity), beta(MultiplicationOp::Annihilator), alpha_ptr(nullptr), beta_ptr(nullptr) {}
    Params(ElementCompute alpha_, ElementCompute beta_) : alpha(alpha_), beta(beta_), alpha_ptr(nullptr), beta_ptr(nullptr) {}
    Params(ElementCompute alpha_) : alpha(alpha_), beta(MultiplicationOp::Annihilator), alpha_ptr(nullptr), beta_ptr(nullptr) {}
    Params(ElementCompute const *alpha_ptr_, ElementCompute const *beta_ptr_)
        : alpha(MultiplicationOp::Identity), beta(MultiplicationOp::Annihilator), alpha_ptr(alpha_ptr_), beta_ptr(beta_ptr_) {}
    Params(ElementCompute const *alpha_ptr_)
        : alpha(MultiplicationOp::Identity), beta(MultiplicationOp::Annihilator), alpha_ptr(alpha_ptr_), beta_ptr(nullptr) {}
  };

  /// Host evaluation with by-value scalars (pointer scalars live on the device).
  explicit SemiringLinearCombination(Params const &p) : alpha_(p.alpha), beta_(p.beta) {}

  /// C is read only if mult(beta, MultOp::Identity) differs from AddOp::Identity.
  bool is_source_needed() const {
    ElementCompute const add_identity = AdditionOp::Identity;
    ElementCompute const mult_identity = MultiplicationOp::Identity;
    return add_identity != MultiplicationOp()(beta_, mult_identity);
  }

  ElementOutput operator()(ElementAccumulator const &accum, ElementOutput const &source) const {
    return AdditionOp()(MultiplicationOp()(alpha_, accum), MultiplicationOp()(beta_, source));
  }
  ElementOutput operator()(ElementAccumulator const &accum) const { return MultiplicationOp()(alpha_, accum); }

 private:
  ElementCompute alpha_, beta_;
};

}  // namespace thread
}  // namespace epilogue
}  // namespace cuasr
