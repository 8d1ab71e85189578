// Runs the C++ split-K models of oracle/include/cuasr/reference/srgemm/host_srgemm_splitk.h (the checker of
// the kernels built from user functors) with the library's own functor types on inputs that
// tests/test_oracle.py regenerates, and prints the results as hexadecimal bit patterns; the Python side
// compares them with the C oracle's split-K models (oracle/host_srgemm.c), which are pinned on their own.
// Host code only (g++).
//   usage: host_splitk_models <parallel|serial> <plustimes|mintimes> <m> <n> <k> <slices>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "cuasr/functional.h"
#include "cuasr/reference/srgemm/host_srgemm_splitk.h"

// value i of stream `seed`: sevenths in [-3, 11.3): products and sums round
static float value(unsigned seed, unsigned i) { return float((i * 37u + seed * 11u + (i >> 3) * 5u) % 101u) / 7.0f - 3.0f; }

template <typename Add, typename Mul> static void run(bool serial, int m, int n, int k, int slices, float alpha, float beta) {
  using Col = cuasr::layout::ColumnMajor;
  using Row = cuasr::layout::RowMajor;
  std::vector<float> A(size_t(m) * k), B(size_t(k) * n), C(size_t(m) * n), D(size_t(m) * n);
  for (size_t i = 0; i < A.size(); ++i) A[i] = value(1, unsigned(i));   // column-major m x k
  for (size_t i = 0; i < B.size(); ++i) B[i] = value(2, unsigned(i));   // row-major k x n
  for (size_t i = 0; i < C.size(); ++i) C[i] = value(3, unsigned(i));   // column-major m x n
  using Model = cuasr::reference::host::SrgemmSplitK<Add, Mul, float, Col, Row, Col>;
  if (serial) Model::serial({m, n, k}, alpha, {A.data(), m}, {B.data(), n}, beta, {C.data(), m}, {D.data(), m}, slices);
  else Model::parallel({m, n, k}, alpha, {A.data(), m}, {B.data(), n}, beta, {C.data(), m}, {D.data(), m}, slices);
  for (float v : D) {
    unsigned bits;
    std::memcpy(&bits, &v, 4);
    std::printf("%08x\n", bits);
  }
}

int main(int argc, char **argv) {
  if (argc != 7) return 2;
  const bool serial = !std::strcmp(argv[1], "serial");
  const int m = std::atoi(argv[3]), n = std::atoi(argv[4]), k = std::atoi(argv[5]), slices = std::atoi(argv[6]);
  if (!std::strcmp(argv[2], "plustimes")) run<cuasr::plus<float>, cuasr::multiplies<float>>(serial, m, n, k, slices, 1.25f, 0.5f);
  else run<cuasr::minimum<float>, cuasr::multiplies<float>>(serial, m, n, k, slices, -1.5f, 1.0f);
  return 0;
}
