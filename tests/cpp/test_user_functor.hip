// device::Srgemm with functors that are none of the library's operators: the kernel is built from the
// functors' operator() (as the reference does for every functor,
// examples/01_userdefined_semiring/userdefined_semiring.cu:56-99), and must reproduce the host reference
// SRGEMM bit for bit -- also for an "add" that is not associative, because every output element is
// accumulated in ascending k like the host loop.  Both split-K forms for such functors
// (device::SrgemmSplitKParallel as in examples/02_splitk_srgemm/splitk_srgemm.cu:44-86, and
// device::Srgemm<..., SplitKSerial = true>) against the CPU models of what the reference's kernels compute,
// on functors whose results depend on where a slice ends.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <array>
#include <vector>

#include "cuasr/gemm/device/srgemm.h"
#include "cuasr/gemm/device/srgemm_splitk_parallel.h"
#include "cuasr/reference/srgemm/host_srgemm.h"
#include "cuasr/reference/srgemm/host_srgemm_splitk.h"

#define HIP_CHECK(x)                                                                                   \
  do {                                                                                                 \
    hipError_t e_ = (x);                                                                               \
    if (e_ != hipSuccess) {                                                                            \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__);               \
      std::exit(2);                                                                                    \
    }                                                                                                  \
  } while (0)

static int g_run = 0, g_fail = 0;
static void check(bool ok, const char *what) {
  ++g_run;
  if (!ok) ++g_fail;
  std::printf("%s %s\n", ok ? "PASS" : "FAIL", what);
}

// a bounded "plus": path lengths saturate at a cap (shortest paths with a horizon)
template <typename T, int N = 1> struct saturating_plus {
  static constexpr T Identity = static_cast<T>(0);
  static constexpr T Annihilator = static_cast<T>(1000);
  __host__ __device__ T operator()(T lhs, T const &rhs) const {
    const T s = lhs + rhs;
    return s > static_cast<T>(1000) ? static_cast<T>(1000) : s;
  }
};
template <typename T, int N> constexpr T saturating_plus<T, N>::Identity;
template <typename T, int N> constexpr T saturating_plus<T, N>::Annihilator;

// keeps the operand of larger magnitude (ties: the right one): not commutative on ties, order matters
template <typename T, int N = 1> struct abs_max {
  static constexpr T Identity = static_cast<T>(0);
  static constexpr T Annihilator = static_cast<T>(0);
  __host__ __device__ T operator()(T lhs, T const &rhs) const { return (lhs < 0 ? -lhs : lhs) > (rhs < 0 ? -rhs : rhs) ? lhs : rhs; }
};
template <typename T, int N> constexpr T abs_max<T, N>::Identity;
template <typename T, int N> constexpr T abs_max<T, N>::Annihilator;

// a decayed sum: not associative, rounds at every step
template <typename T, int N = 1> struct leaky_plus {
  static constexpr T Identity = static_cast<T>(0);
  static constexpr T Annihilator = static_cast<T>(0);
  __host__ __device__ T operator()(T lhs, T const &rhs) const { return lhs + static_cast<T>(0.75) * rhs; }
};
template <typename T, int N> constexpr T leaky_plus<T, N>::Identity;
template <typename T, int N> constexpr T leaky_plus<T, N>::Annihilator;

template <typename Add, typename Mul, typename T, typename LA, typename LB, typename LC>
static void run_case(int m, int n, int k, T alpha, T beta, unsigned seed, const char *what) {
  using Op = cuasr::gemm::device::Srgemm<Add, Mul, T, LA, T, LB, T, LC, T>;
  static_assert(Op::kUserFunctors, "this test is about functors the library has no operator for");
  const bool a_col = LA::kAbiTag == CUASR_AMD_COLUMN_MAJOR, b_col = LB::kAbiTag == CUASR_AMD_COLUMN_MAJOR,
             c_col = LC::kAbiTag == CUASR_AMD_COLUMN_MAJOR;
  const int lda = (a_col ? m : k) + 3, ldb = (b_col ? k : n) + 1, ldc = (c_col ? m : n) + 2;
  std::vector<T> A((size_t)lda * (a_col ? k : m)), B((size_t)ldb * (b_col ? n : k)), C((size_t)ldc * (c_col ? n : m)), D(C.size()), R(C.size());
  std::mt19937 rng(seed);
  std::uniform_int_distribution<int> dist(-40, 40);
  for (auto &v : A) v = static_cast<T>(dist(rng)) / static_cast<T>(std::is_integral<T>::value ? 1 : 8);
  for (auto &v : B) v = static_cast<T>(dist(rng)) / static_cast<T>(std::is_integral<T>::value ? 1 : 8);
  for (auto &v : C) v = static_cast<T>(dist(rng)) / static_cast<T>(std::is_integral<T>::value ? 1 : 8);
  D.assign(D.size(), static_cast<T>(-77));
  R = D;
  T *dA, *dB, *dC, *dD;
  HIP_CHECK(hipMalloc(&dA, A.size() * sizeof(T)));
  HIP_CHECK(hipMalloc(&dB, B.size() * sizeof(T)));
  HIP_CHECK(hipMalloc(&dC, C.size() * sizeof(T)));
  HIP_CHECK(hipMalloc(&dD, D.size() * sizeof(T)));
  HIP_CHECK(hipMemcpy(dA, A.data(), A.size() * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dB, B.data(), B.size() * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dC, C.data(), C.size() * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dD, D.data(), D.size() * sizeof(T), hipMemcpyHostToDevice));
  typename Op::Arguments args({m, n, k}, {dA, lda}, {dB, ldb}, {dC, ldc}, {dD, ldc}, {alpha, beta});
  Op op;
  const cuasr::Status st = op(args);
  HIP_CHECK(hipDeviceSynchronize());
  HIP_CHECK(hipMemcpy(D.data(), dD, D.size() * sizeof(T), hipMemcpyDeviceToHost));
  cuasr::reference::host::Srgemm<Add, Mul, T, LA, T, LB, T, LC, T, T> ref;
  ref({m, n, k}, alpha, {A.data(), lda}, {B.data(), ldb}, beta, {C.data(), ldc}, {R.data(), ldc}, Add::Identity);
  char name[256];
  std::snprintf(name, sizeof name, "%s %dx%dx%d", what, m, n, k);
  check(st == cuasr::Status::kSuccess && std::memcmp(D.data(), R.data(), D.size() * sizeof(T)) == 0, name);
  HIP_CHECK(hipFree(dA));
  HIP_CHECK(hipFree(dB));
  HIP_CHECK(hipFree(dC));
  HIP_CHECK(hipFree(dD));
}

// SERIAL = false: device::SrgemmSplitKParallel; true: device::Srgemm with SplitKSerial (every tuning parameter spelled out,
// as a caller of the reference has to in order to reach the last one)
template <typename Add, typename Mul, typename T, typename LA, typename LB, typename LC, bool SERIAL>
static void run_splitk_case(int m, int n, int k, T alpha, T beta, int slices, unsigned seed, const char *what) {
  using Config = cuasr::gemm::device::DefaultSemiRingConfiguration<T, T, T, T, cuasr::arch::OpClassSimt, Add, Mul, cuasr::arch::Sm50>;
  using Parallel = cuasr::gemm::device::SrgemmSplitKParallel<Add, Mul, T, LA, T, LB, T, LC, T>;
  using Serial = cuasr::gemm::device::Srgemm<Add, Mul, T, LA, T, LB, T, LC, T, cuasr::arch::OpClassSimt, cuasr::arch::Sm50,
                                             typename Config::ThreadblockShape, typename Config::WarpShape,
                                             typename Config::InstructionShape, typename Config::EpilogueOutputOp,
                                             cuasr::gemm::threadblock::GemmIdentityThreadblockSwizzle<>, Config::kStages, 1, 1, true>;
  using Op = typename std::conditional<SERIAL, Serial, Parallel>::type;
  static_assert(Op::kUserFunctors, "this test is about functors the library has no operator for");
  const bool a_col = LA::kAbiTag == CUASR_AMD_COLUMN_MAJOR, b_col = LB::kAbiTag == CUASR_AMD_COLUMN_MAJOR,
             c_col = LC::kAbiTag == CUASR_AMD_COLUMN_MAJOR;
  const int lda = (a_col ? m : k) + 4, ldb = (b_col ? k : n) + 2, ldc = (c_col ? m : n) + 1;
  std::vector<T> A((size_t)lda * (a_col ? k : m)), B((size_t)ldb * (b_col ? n : k)), C((size_t)ldc * (c_col ? n : m)), D(C.size()), R(C.size());
  std::mt19937 rng(seed);
  std::uniform_int_distribution<int> dist(-40, 40);
  for (auto &v : A) v = static_cast<T>(dist(rng)) / static_cast<T>(std::is_integral<T>::value ? 1 : 8);
  for (auto &v : B) v = static_cast<T>(dist(rng)) / static_cast<T>(std::is_integral<T>::value ? 1 : 8);
  for (auto &v : C) v = static_cast<T>(dist(rng)) / static_cast<T>(std::is_integral<T>::value ? 1 : 8);
  D.assign(D.size(), static_cast<T>(-77));
  R = D;
  T *dA, *dB, *dC, *dD;
  HIP_CHECK(hipMalloc(&dA, A.size() * sizeof(T)));
  HIP_CHECK(hipMalloc(&dB, B.size() * sizeof(T)));
  HIP_CHECK(hipMalloc(&dC, C.size() * sizeof(T)));
  HIP_CHECK(hipMalloc(&dD, D.size() * sizeof(T)));
  HIP_CHECK(hipMemcpy(dA, A.data(), A.size() * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dB, B.data(), B.size() * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dC, C.data(), C.size() * sizeof(T), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dD, D.data(), D.size() * sizeof(T), hipMemcpyHostToDevice));
  typename Op::Arguments args({m, n, k}, {dA, lda}, {dB, ldb}, {dC, ldc}, {dD, ldc}, {alpha, beta}, slices);
  const size_t bytes = Op::get_workspace_size(args);
  bool ok = bytes == ((SERIAL && slices == 1) ? 0 : sizeof(T) * (size_t)m * n * slices);
  cutlass::device_memory::allocation<uint8_t> workspace(bytes + 16);   // (never empty, so that a parallel run with one slice has one)
  Op op;
  ok = ok && op.initialize(args, workspace.get()) == cuasr::Status::kSuccess;
  if (slices > 1 || !SERIAL) ok = ok && Op().initialize(args, nullptr) == cuasr::Status::kErrorWorkspaceNull;
  ok = ok && op.run() == cuasr::Status::kSuccess;
  HIP_CHECK(hipDeviceSynchronize());
  HIP_CHECK(hipMemcpy(D.data(), dD, D.size() * sizeof(T), hipMemcpyDeviceToHost));
  using Model = cuasr::reference::host::SrgemmSplitK<Add, Mul, T, LA, LB, LC>;
  if (SERIAL) Model::serial({m, n, k}, alpha, {A.data(), lda}, {B.data(), ldb}, beta, {C.data(), ldc}, {R.data(), ldc}, slices);
  else Model::parallel({m, n, k}, alpha, {A.data(), lda}, {B.data(), ldb}, beta, {C.data(), ldc}, {R.data(), ldc}, slices);
  char name[256];
  std::snprintf(name, sizeof name, "%s split-K %s %dx%dx%d, %d slices", SERIAL ? "serial" : "parallel", what, m, n, k, slices);
  check(ok && std::memcmp(D.data(), R.data(), D.size() * sizeof(T)) == 0, name);
  HIP_CHECK(hipFree(dA));
  HIP_CHECK(hipFree(dB));
  HIP_CHECK(hipFree(dC));
  HIP_CHECK(hipFree(dD));
}

// the reference example's own user functor, spelled as there (no Annihilator: an addition needs none):
// examples/01_userdefined_semiring/userdefined_semiring.cu:56-66
namespace {
template <typename T, int N = 1> struct example_xor {
  static T constexpr Identity = static_cast<T>(false);
  __host__ __device__ T operator()(T lhs, T const &rhs) const {
    lhs ^= rhs;
    return lhs;
  }
};
}  // namespace

int main() {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count == 0) {
    std::printf("no GPU\n");
    return 1;
  }
  using Col = cuasr::layout::ColumnMajor;
  using Row = cuasr::layout::RowMajor;
  // (the last two span several tiles of the kernel's XCD-aware tile order, whole and ragged)
  const int shapes[][3] = {{64, 64, 64}, {1, 1, 1}, {65, 63, 17}, {200, 130, 301}, {7, 300, 33}, {509, 510, 23},
                           {1024, 512, 40}, {390, 1100, 19}};
  for (auto &s : shapes) {
    // library add, user mult: bounded shortest paths on integers
    run_case<cuasr::minimum<int32_t>, saturating_plus<int32_t>, int32_t, Col, Col, Col>(s[0], s[1], s[2], 0, 0, 11, "min / saturating-plus i32 ccc");
    run_case<cuasr::minimum<int32_t>, saturating_plus<int32_t>, int32_t, Row, Col, Row>(s[0], s[1], s[2], 5, 1000, 12, "min / saturating-plus i32 rcr, beta = annihilator");
    // user add (order-dependent on ties), library mult
    run_case<abs_max<float>, cuasr::multiplies<float>, float, Col, Row, Col>(s[0], s[1], s[2], 1.0f, 1.0f, 13, "abs-max / times f32 crc");
    run_case<abs_max<float>, cuasr::multiplies<float>, float, Row, Row, Row>(s[0], s[1], s[2], -2.0f, 0.5f, 14, "abs-max / times f32 rrr");
    // both user-defined, a non-associative add in double: only the host's own order gives these bits
    run_case<leaky_plus<double>, saturating_plus<double>, double, Col, Col, Row>(s[0], s[1], s[2], 1.5, 0.5, 15, "leaky-plus / saturating-plus f64 ccr");
  }
  // outputs of 512 full-size tiles and more (below that the launcher takes the quarter-size tile): whole, and with ragged edges
  run_case<abs_max<float>, cuasr::multiplies<float>, float, Col, Row, Col>(2048, 4096, 24, 1.0f, 1.0f, 31, "abs-max / times f32 crc, full-size tiles");
  run_case<abs_max<float>, cuasr::multiplies<float>, float, Row, Col, Row>(2100, 4000, 35, -2.0f, 0.5f, 32, "abs-max / times f32 rcr, full-size tiles, ragged");
  run_case<abs_max<float>, cuasr::multiplies<float>, float, Row, Row, Row>(2048, 4096, 17, 1.0f, 1.0f, 33, "abs-max / times f32 rrr, full-size tiles");
  run_case<abs_max<float>, cuasr::multiplies<float>, float, Col, Col, Col>(2101, 4001, 18, 1.0f, 1.0f, 34, "abs-max / times f32 ccc, full-size tiles, odd extents");
  run_case<leaky_plus<double>, saturating_plus<double>, double, Col, Col, Row>(2048, 2048, 33, 1.5, 0.5, 35, "leaky-plus / saturating-plus f64 ccr, full-size tiles");
  run_case<leaky_plus<double>, saturating_plus<double>, double, Row, Col, Col>(2050, 2100, 20, 1.5, 0.5, 36, "leaky-plus / saturating-plus f64 rcc, full-size tiles, ragged");
  run_splitk_case<abs_max<float>, cuasr::multiplies<float>, float, Row, Col, Col, false>(2048, 2048, 70, -2.0f, 0.5f, 2, 37, "abs-max / times f32 rcc, full-size tiles");
  run_splitk_case<leaky_plus<double>, saturating_plus<double>, double, Col, Col, Row, true>(1024, 2048, 50, 1.5, 0.5, 3, 38, "leaky-plus / saturating-plus f64 ccr, full-size tiles");

  // xor-and on 0 / 1 integers with the example's own addition functor (the multiplication is the library's)
  run_case<example_xor<int>, cuasr::binary_and<int>, int, Row, Row, Row>(512, 512, 512, 1, 1, 16, "example xor / binary_and i32 rrr");
  run_case<example_xor<int>, cuasr::binary_and<int>, int, Row, Row, Row>(130, 70, 33, 1, 0, 17, "example xor / binary_and i32 rrr, beta = 0");

  // split-K, both forms, slices 1, 2, 3, 8 (test/device/testbed.h:322-338 sweeps these), on functor pairs whose
  // bits depend on the slice boundaries: a non-associative add, and a saturating product under a scaling alpha
  for (int slices : {1, 2, 3, 8}) {
    for (auto &s : {std::array<int, 3>{128, 128, 4096}, std::array<int, 3>{65, 63, 100}, std::array<int, 3>{200, 130, 301}, std::array<int, 3>{7, 33, 5}}) {
      run_splitk_case<leaky_plus<double>, saturating_plus<double>, double, Col, Col, Row, false>(s[0], s[1], s[2], 1.5, 0.5, slices, 21, "leaky-plus / saturating-plus f64 ccr");
      run_splitk_case<leaky_plus<double>, saturating_plus<double>, double, Col, Col, Row, true>(s[0], s[1], s[2], 1.5, 0.5, slices, 22, "leaky-plus / saturating-plus f64 ccr");
      run_splitk_case<abs_max<float>, cuasr::multiplies<float>, float, Row, Col, Col, false>(s[0], s[1], s[2], -2.0f, 0.5f, slices, 23, "abs-max / times f32 rcc");
      run_splitk_case<abs_max<float>, cuasr::multiplies<float>, float, Row, Col, Col, true>(s[0], s[1], s[2], -2.0f, 0.5f, slices, 24, "abs-max / times f32 rcc");
      run_splitk_case<cuasr::minimum<int32_t>, saturating_plus<int32_t>, int32_t, Col, Row, Row, false>(s[0], s[1], s[2], 5, 1000, slices, 25, "min / saturating-plus i32 crr, beta = annihilator");
      run_splitk_case<cuasr::minimum<int32_t>, saturating_plus<int32_t>, int32_t, Col, Row, Row, true>(s[0], s[1], s[2], 5, 0, slices, 26, "min / saturating-plus i32 crr");
    }
  }
  // more slices than k-tiles: the parallel form leaves every slice but the last empty, the serial form the trailing ones
  run_splitk_case<leaky_plus<double>, saturating_plus<double>, double, Col, Col, Row, false>(40, 24, 20, 1.5, 0.5, 16, 27, "leaky-plus / saturating-plus f64 ccr");
  run_splitk_case<leaky_plus<double>, saturating_plus<double>, double, Col, Col, Row, true>(40, 24, 20, 1.5, 0.5, 16, 28, "leaky-plus / saturating-plus f64 ccr");

  // the run-time checks that do not depend on the functors
  {
    using Op = cuasr::gemm::device::Srgemm<abs_max<float>, cuasr::multiplies<float>, float, Col, float, Col, float, Col, float>;
    float *d = nullptr;
    HIP_CHECK(hipMalloc(&d, 64 * 64 * 4));
    typename Op::Arguments bad_ld({64, 64, 64}, {d, 10}, {d, 64}, {d, 64}, {d, 64}, {1.0f, 1.0f});
    check(Op::can_implement(bad_ld) == cuasr::Status::kErrorInvalidProblem, "leading dimension smaller than the extent is refused");
    typename Op::Arguments split({64, 64, 64}, {d, 64}, {d, 64}, {d, 64}, {d, 64}, {1.0f, 1.0f}, 4);
    check(Op::can_implement(split) == cuasr::Status::kErrorInvalidProblem, "split_k_slices > 1 is refused (device/srgemm.h:198-200)");
    Op op;
    check(op.run() == cuasr::Status::kErrorInternal, "run before initialize is refused");
    HIP_CHECK(hipFree(d));
  }
  std::printf("%d checks, %d failed\n", g_run, g_fail);
  return g_fail ? 1 : 0;
}
