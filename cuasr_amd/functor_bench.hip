// Throughput of the kernels device::Srgemm builds from user functors (cuasr/gemm/kernel/functor_srgemm.h),
// measured the way a user gets them: functors defined in this translation unit, compiled by hipcc with the
// flags the library's own objects use.  Each functor pair runs an N^3 SRGEMM (column-major A, row-major B,
// column-major C and D, alpha = beta = one, as the reference's min-plus example,
// examples/00_minplus_srgemm/minplus_srgemm.cu:22-61) and one split-K case; pairs that compute min-plus are
// also compared bit for bit with the library's tuned min-plus kernel on the same operands.
// Prints one JSON object per line.   usage: functor_bench [N = 4096] [steps = 10] [warmup = 5]
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <vector>

#include "cuasr/gemm/device/srgemm.h"
#include "cuasr/gemm/device/srgemm_splitk_parallel.h"

#define HIP_OK(x)                                                                        \
  do {                                                                                   \
    hipError_t e_ = (x);                                                                 \
    if (e_ != hipSuccess) {                                                              \
      std::fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      std::exit(2);                                                                      \
    }                                                                                    \
  } while (0)

// ---- user functors: none of them has a cuasr::op_tag, so every kernel below is built from these bodies ----
// minimum through the math library: maps to the hardware minimum, which the compiler can fold in threes
template <typename T, int N = 1> struct fmin_op {
  static constexpr T Identity = std::numeric_limits<T>::infinity();
  static constexpr T Annihilator = -std::numeric_limits<T>::infinity();
  __host__ __device__ T operator()(T lhs, T const &rhs) const { return fminf(lhs, rhs); }
};
// minimum spelled as the reference's functor spells it (include/cuasr/functional.h:132): a comparison and a select
template <typename T, int N = 1> struct ternary_min {
  static constexpr T Identity = std::numeric_limits<T>::infinity();
  static constexpr T Annihilator = -std::numeric_limits<T>::infinity();
  __host__ __device__ T operator()(T lhs, T const &rhs) const { return rhs < lhs ? rhs : lhs; }
};
template <typename T, int N = 1> struct user_plus {
  static constexpr T Identity = static_cast<T>(0);
  static constexpr T Annihilator = std::numeric_limits<T>::infinity();
  __host__ __device__ T operator()(T lhs, T const &rhs) const { return lhs + rhs; }
};
// path lengths that saturate at a horizon: no library operator computes this
template <typename T, int N = 1> struct saturating_plus {
  static constexpr T Identity = static_cast<T>(0);
  static constexpr T Annihilator = static_cast<T>(1000);
  __host__ __device__ T operator()(T lhs, T const &rhs) const {
    const T s = lhs + rhs;
    return s > static_cast<T>(1000) ? static_cast<T>(1000) : s;
  }
};

static unsigned long long mix(unsigned long long &s) {
  unsigned long long z = (s += 0x9e3779b97f4a7c15ull);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}
static void fill(std::vector<float> &v, unsigned long long seed, float lo, float hi) {
  for (auto &x : v) x = lo + (hi - lo) * float(mix(seed) >> 40) * (1.0f / 16777216.0f);
}

struct Buffers {
  float *A, *B, *C, *D, *R;
};

template <typename Add, typename Mul> static void run_pair(const char *name, int n, int steps, int warmup, const Buffers &b, bool is_min_plus) {
  using Col = cuasr::layout::ColumnMajor;
  using Row = cuasr::layout::RowMajor;
  using Op = cuasr::gemm::device::Srgemm<Add, Mul, float, Col, float, Row, float, Col, float>;
  static_assert(Op::kUserFunctors, "the point of this program");
  typename Op::Arguments args({n, n, n}, {b.A, n}, {b.B, n}, {b.C, n}, {b.D, n}, {Mul::Identity, Mul::Identity});
  Op op;
  if (op.initialize(args) != cuasr::Status::kSuccess) std::exit(3);
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  for (int i = 0; i < warmup; ++i) op.run();
  HIP_OK(hipEventRecord(e0, nullptr));
  for (int i = 0; i < steps; ++i) op.run();
  HIP_OK(hipEventRecord(e1, nullptr));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  ms /= steps;
  int same = -1;
  if (is_min_plus) {
    // the library's tuned kernel on the same operands
    using Tuned = cuasr::gemm::device::Srgemm<cuasr::inf::minimum<float>, cuasr::plus<float>, float, Col, float, Row, float, Col, float>;
    typename Tuned::Arguments targs({n, n, n}, {b.A, n}, {b.B, n}, {b.C, n}, {b.R, n}, {0.0f, 0.0f});
    Tuned tuned;
    if (tuned(targs) != cuasr::Status::kSuccess) std::exit(4);
    HIP_OK(hipDeviceSynchronize());
    std::vector<float> d(size_t(n) * n), r(size_t(n) * n);
    HIP_OK(hipMemcpy(d.data(), b.D, d.size() * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(r.data(), b.R, r.size() * 4, hipMemcpyDeviceToHost));
    same = std::memcmp(d.data(), r.data(), d.size() * 4) == 0;
  }
  std::printf("{\"workload\": \"functor srgemm %s f32 %d^3 (A column-major, B row-major, C column-major, alpha = beta = one)\", "
              "\"ms\": %.4f, \"tops\": %.2f, \"frac_of_fp32_vector_peak\": %.4f, \"bit_identical_to_tuned_min_plus\": %s}\n",
              name, n, ms, 2.0 * n * n * double(n) / (ms * 1e9), 2.0 * n * n * double(n) / (ms * 1e9) / 157.3,
              same < 0 ? "null" : same ? "true" : "false");
  std::fflush(stdout);
}

// the reference's split-K example shape (examples/02_splitk_srgemm/splitk_srgemm.cu:44-86: A row-major, B column-major)
template <typename Add, typename Mul> static void run_splitk(const char *name, int m, int k, int slices, int steps, int warmup, const Buffers &b) {
  using Col = cuasr::layout::ColumnMajor;
  using Row = cuasr::layout::RowMajor;
  using Op = cuasr::gemm::device::SrgemmSplitKParallel<Add, Mul, float, Row, float, Col, float, Row, float>;
  typename Op::Arguments args({m, m, k}, {b.A, k}, {b.B, k}, {b.C, m}, {b.D, m}, {Mul::Identity, Mul::Annihilator}, slices);
  cutlass::device_memory::allocation<uint8_t> workspace(Op::get_workspace_size(args));
  Op op;
  if (op.initialize(args, workspace.get()) != cuasr::Status::kSuccess) std::exit(5);
  hipEvent_t e0, e1;
  HIP_OK(hipEventCreate(&e0));
  HIP_OK(hipEventCreate(&e1));
  for (int i = 0; i < warmup; ++i) op.run();
  HIP_OK(hipEventRecord(e0, nullptr));
  for (int i = 0; i < steps; ++i) op.run();
  HIP_OK(hipEventRecord(e1, nullptr));
  HIP_OK(hipEventSynchronize(e1));
  float ms = 0;
  HIP_OK(hipEventElapsedTime(&ms, e0, e1));
  ms /= steps;
  std::printf("{\"workload\": \"functor split-K %s f32 %dx%dx%d, %d slices\", \"ms\": %.4f, \"tops\": %.2f}\n", name, m, m, k, slices, ms,
              2.0 * m * m * double(k) / (ms * 1e9));
  std::fflush(stdout);
}

int main(int argc, char **argv) {
  const int n = argc > 1 ? std::atoi(argv[1]) : 4096, steps = argc > 2 ? std::atoi(argv[2]) : 10, warmup = argc > 3 ? std::atoi(argv[3]) : 5;
  if (n < 256 || n % 4) return 2;
  const size_t elems = size_t(n) * n > size_t(256) * 65536 ? size_t(n) * n : size_t(256) * 65536;
  std::vector<float> h(elems);
  Buffers b;
  HIP_OK(hipMalloc(&b.A, elems * 4));
  HIP_OK(hipMalloc(&b.B, elems * 4));
  HIP_OK(hipMalloc(&b.C, elems * 4));
  HIP_OK(hipMalloc(&b.D, elems * 4));
  HIP_OK(hipMalloc(&b.R, elems * 4));
  fill(h, 1, 0.0f, 10.0f);
  HIP_OK(hipMemcpy(b.A, h.data(), elems * 4, hipMemcpyHostToDevice));
  fill(h, 2, 0.0f, 10.0f);
  HIP_OK(hipMemcpy(b.B, h.data(), elems * 4, hipMemcpyHostToDevice));
  fill(h, 3, 0.0f, 30.0f);
  HIP_OK(hipMemcpy(b.C, h.data(), elems * 4, hipMemcpyHostToDevice));
  run_pair<fmin_op<float>, user_plus<float>>("fmin / user plus (min-plus through the math library's fminf)", n, steps, warmup, b, true);
  run_pair<ternary_min<float>, user_plus<float>>("ternary min / user plus (min-plus as a comparison and a select)", n, steps, warmup, b, true);
  run_pair<fmin_op<float>, saturating_plus<float>>("fmin / saturating plus (no library operator)", n, steps, warmup, b, false);
  // a size whose full-size tiles would leave three quarters of the chip idle: the quarter-size tile
  run_pair<fmin_op<float>, user_plus<float>>("fmin / user plus (min-plus through the math library's fminf)", 1024, 4 * steps, 4 * warmup, b, true);
  run_splitk<fmin_op<float>, user_plus<float>>("fmin / user plus", 256, 65536, 8, steps, warmup, b);
  run_splitk<fmin_op<float>, user_plus<float>>("fmin / user plus", 256, 65536, 64, steps, warmup, b);
  return 0;
}
