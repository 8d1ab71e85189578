// cuasr::reference::host::Srgemm for C++ test programs -- TEST INFRASTRUCTURE,
// lives under oracle/ and is never included by the library.
//
// A C++ restatement of tools/include/cuasr/reference/srgemm/host_srgemm.h:33-113:
// accum starts at add_identity, accum = add(mult(a, b), accum) for k ascending,
// D = add(mult(alpha, accum), mult(beta, C)), C always read.  Same call
// signature, so the reference's test and example code reads unchanged.
#pragma once
#include "cuasr/functional.h"

namespace cuasr {
namespace reference {
namespace host {

template <typename AdditionOp, typename MultiplicationOp, typename ElementA, typename LayoutA, typename ElementB,
          typename LayoutB, typename ElementC, typename LayoutC, typename ScalarType, typename ComputeType,
          typename EpilogueOp = void>
struct Srgemm {
  void operator()(gemm::GemmCoord problem_size, ComputeType alpha, TensorRef<ElementA, LayoutA> tensor_a,
                  TensorRef<ElementB, LayoutB> tensor_b, ComputeType beta, TensorRef<ElementC, LayoutC> tensor_c,
                  TensorRef<ElementC, LayoutC> tensor_d, ComputeType add_identity) const {
    AdditionOp add_op;
    MultiplicationOp mult_op;
    for (int row = 0; row < problem_size.m(); ++row) {
      for (int col = 0; col < problem_size.n(); ++col) {
        ComputeType accum = add_identity;
        for (int k = 0; k < problem_size.k(); ++k) {
          ComputeType a = static_cast<ComputeType>(tensor_a.at(MatrixCoord(row, k)));
          ComputeType b = static_cast<ComputeType>(tensor_b.at(MatrixCoord(k, col)));
          accum = add_op(mult_op(a, b), accum);
        }
        ComputeType c = static_cast<ComputeType>(tensor_c.at(MatrixCoord(row, col)));
        tensor_d.at(MatrixCoord(row, col)) = static_cast<ElementC>(add_op(mult_op(alpha, accum), mult_op(beta, c)));
      }
    }
  }
};

}  // namespace host
}  // namespace reference
}  // namespace cuasr
