// CPU models of the reference's two split-K forms for ANY functor pair -- TEST INFRASTRUCTURE, lives under
// oracle/ and is never included by the library.  The reference has no host split-K; what its device code
// computes is restated here as plain loops:
//
//   SrgemmSplitKParallel  (include/cuasr/gemm/kernel/srgemm_splitk_parallel.h:86-89, :136-142,
//                          include/cuasr/reduction/kernel/reduce_split_k.h:162-227,
//                          include/cuasr/reduction/thread/reduction_operators.h:74-86)
//       slice extent ks = ((K / tbk) / S) * tbk, slice z covers [z * ks, (z + 1) * ks), the last slice runs to K;
//       partial[z] = the host loop's accum over that range, from AddOp::Identity;
//       acc = AddOp::Identity; acc = add(acc, partial[z]) for z ascending;
//       source = C where needed, else AddOp::Identity;  D = add(mult(alpha, acc), mult(beta, source)).
//   SrgemmSplitKSerial    (include/cuasr/gemm/kernel/srgemm.h:97-100, :184-189, :249-320,
//                          include/cuasr/gemm/epilogue/thread/semiring_linear_combination.h:118-134, :152-183)
//       slice extent ks = ceil(ceil(K / tbk) / S) * tbk, slice z covers [min(K, z * ks), min(K, (z + 1) * ks));
//       slice 0: D = epilogue(alpha, accum_0, beta, C); slice z > 0: D = epilogue(alpha, accum_z, MultOp::Identity, D);
//       epilogue(a, x, b, s) = add(mult(a, x), mult(b, s)) when AddOp::Identity != mult(b, MultOp::Identity), else mult(a, x).
//   Inside a slice the host reference's order is kept: accum = add(mult(a, b), accum), k ascending
//   (tools/include/cuasr/reference/srgemm/host_srgemm.h:75-91).
//
// tbk is the k-tile depth of the reference's threadblock shape: 8 in every default configuration.
//
// Parity status: pinned by tests/test_oracle.py::test_cpp_splitk_models_agree_with_the_c_oracle (the same
// models in oracle/host_srgemm.c, themselves pinned against literal pure-Python chains, on plus-times with
// non-integer data and on min-times with a negative alpha, where the bits depend on the slice boundaries).
#pragma once
#include <vector>

#include "host_srgemm.h"

namespace cuasr {
namespace reference {
namespace host {

template <typename AdditionOp, typename MultiplicationOp, typename Element, typename LayoutA, typename LayoutB, typename LayoutC>
struct SrgemmSplitK {
  static Element partial(gemm::GemmCoord problem, TensorRef<Element, LayoutA> a, TensorRef<Element, LayoutB> b, int row, int col,
                         long long k_begin, long long k_end) {
    AdditionOp add_op;
    MultiplicationOp mult_op;
    Element accum = AdditionOp::Identity;
    for (long long k = k_begin; k < k_end && k < problem.k(); ++k)
      accum = add_op(mult_op(a.at(MatrixCoord(row, int(k))), b.at(MatrixCoord(int(k), col))), accum);
    return accum;
  }
  static bool source_needed(Element beta) { return !(AdditionOp::Identity == MultiplicationOp()(beta, MultiplicationOp::Identity)); }

  /// the two-kernel parallel form
  static void parallel(gemm::GemmCoord problem, Element alpha, TensorRef<Element, LayoutA> a, TensorRef<Element, LayoutB> b,
                       Element beta, TensorRef<Element, LayoutC> c, TensorRef<Element, LayoutC> d, int slices, int tbk = 8) {
    AdditionOp add_op;
    MultiplicationOp mult_op;
    const long long K = problem.k(), ks = ((K / tbk) / slices) * tbk;
    for (int row = 0; row < problem.m(); ++row)
      for (int col = 0; col < problem.n(); ++col) {
        Element acc = AdditionOp::Identity;
        for (int z = 0; z < slices; ++z)
          acc = add_op(acc, partial(problem, a, b, row, col, z * ks, z + 1 == slices ? K : (z + 1) * ks));
        const Element source = source_needed(beta) ? c.at(MatrixCoord(row, col)) : Element(AdditionOp::Identity);
        d.at(MatrixCoord(row, col)) = add_op(mult_op(alpha, acc), mult_op(beta, source));
      }
  }

  /// the serial form: the slices' epilogues one after the other
  static void serial(gemm::GemmCoord problem, Element alpha, TensorRef<Element, LayoutA> a, TensorRef<Element, LayoutB> b,
                     Element beta, TensorRef<Element, LayoutC> c, TensorRef<Element, LayoutC> d, int slices, int tbk = 8) {
    AdditionOp add_op;
    MultiplicationOp mult_op;
    const long long K = problem.k(), iterations = (K + tbk - 1) / tbk, ks = ((iterations + slices - 1) / slices) * tbk;
    auto epilogue = [&](Element al, Element x, Element be, Element s) {
      return source_needed(be) ? add_op(mult_op(al, x), mult_op(be, s)) : mult_op(al, x);
    };
    for (int row = 0; row < problem.m(); ++row)
      for (int col = 0; col < problem.n(); ++col) {
        Element out = epilogue(alpha, partial(problem, a, b, row, col, 0, ks), beta,
                               source_needed(beta) ? c.at(MatrixCoord(row, col)) : Element());
        for (int z = 1; z < slices; ++z)
          out = epilogue(alpha, partial(problem, a, b, row, col, z * ks, (z + 1) * ks), MultiplicationOp::Identity, out);
        d.at(MatrixCoord(row, col)) = out;
      }
  }
};

}  // namespace host
}  // namespace reference
}  // namespace cuasr
