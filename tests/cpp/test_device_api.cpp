// GPU test of the C++ operator API (cuasr::gemm::device::Srgemm and
// SrgemmSplitKParallel) written the way the reference's own tests and examples
// use it: the testbed sweep (test/device/testbed.h:268-361: m in {1,509},
// n in {1,510}, k in {1,23}, integer-valued inputs in [-8,8], (0,0) forced to
// 1, alpha = Mult::Identity, beta = Mult::Annihilator, bit-exact against the
// host reference), example 00 (min-plus), example 01 (user-defined xor-and),
// example 02 (split-K equals non-split), and the regress known-answer vector.
// Prints one line per check; exit status is the number of failures.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "cuasr/gemm/device/srgemm.h"
#include "cuasr/gemm/device/srgemm_splitk_parallel.h"
#include "cuasr/reference/srgemm/host_srgemm.h"

using cuasr::Status;
using cuasr::layout::ColumnMajor;
using cuasr::layout::RowMajor;

static int g_fail = 0, g_run = 0;
#define HIP_OK(x)                                                                \
  do {                                                                           \
    hipError_t e_ = (x);                                                         \
    if (e_ != hipSuccess) {                                                      \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(99);                                                             \
    }                                                                            \
  } while (0)

static void report(bool ok, const char *what) {
  ++g_run;
  if (!ok) ++g_fail;
  std::printf("%s %s\n", ok ? "PASS" : "FAIL", what);
  std::fflush(stdout);
}

// splitmix64: the same generator the Python tests use
static uint64_t mix(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
template <typename T> static void fill_int(std::vector<T> &v, uint64_t seed, int lo, int hi) {
  for (size_t i = 0; i < v.size(); ++i) v[i] = static_cast<T>(lo + int(mix(seed * 0x9E3779B97F4A7C15ull + i + 1) % uint64_t(hi - lo + 1)));
}
template <typename T> static void fill_unit(std::vector<T> &v, uint64_t seed, double lo, double hi) {
  for (size_t i = 0; i < v.size(); ++i)
    v[i] = static_cast<T>(lo + (hi - lo) * double(mix(seed * 0x9E3779B97F4A7C15ull + i + 1) >> 40) / 16777216.0);
}

template <typename T> struct DeviceBuf {
  T *p = nullptr;
  size_t n = 0;
  explicit DeviceBuf(size_t count) : n(count) { HIP_OK(hipMalloc(reinterpret_cast<void **>(&p), (count ? count : 1) * sizeof(T))); }
  DeviceBuf(std::vector<T> const &h) : DeviceBuf(h.size()) { upload(h); }
  ~DeviceBuf() { (void)hipFree(p); }
  void upload(std::vector<T> const &h) { HIP_OK(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
  std::vector<T> download() const {
    std::vector<T> h(n);
    HIP_OK(hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
};

template <typename L> static long long ld_of(int rows, int cols) { return std::is_same<L, ColumnMajor>::value ? rows : cols; }

// one testbed case: device operator vs host reference, bit-exact
template <typename Add, typename Mul, typename T, typename LA, typename LB, typename LC, bool SERIAL = false>
static bool testbed_case(int m, int n, int k, T alpha, T beta, int slices = 1) {
  using Plain = cuasr::gemm::device::Srgemm<Add, Mul, T, LA, T, LB, T, LC, T>;
  using Op = cuasr::gemm::device::Srgemm<Add, Mul, T, LA, T, LB, T, LC, T, typename Plain::OperatorClass,
                                         typename Plain::ArchTag, typename Plain::ThreadblockShape, typename Plain::WarpShape,
                                         typename Plain::InstructionShape, typename Plain::EpilogueOutputOp,
                                         typename Plain::ThreadblockSwizzle, Plain::kStages, 1, 1, SERIAL>;
  const long long lda = ld_of<LA>(m, k), ldb = ld_of<LB>(k, n), ldc = ld_of<LC>(m, n);
  std::vector<T> A(size_t(m) * k), B(size_t(k) * n), C(size_t(m) * n), D(size_t(m) * n, T(0)), R(size_t(m) * n, T(0));
  fill_int(A, 2019, -8, 8);
  fill_int(B, 2018, -8, 8);
  fill_int(C, 2017, -8, 8);
  A[0] = B[0] = C[0] = T(1);  // as the reference testbed does (testbed.h:142-144)
  DeviceBuf<T> dA(A), dB(B), dC(C), dD(D);
  typename Op::Arguments args({m, n, k}, {dA.p, lda}, {dB.p, ldb}, {dC.p, ldc}, {dD.p, ldc}, {alpha, beta}, slices);
  Op op;
  if (Op::can_implement(args) != Status::kSuccess) return false;
  DeviceBuf<uint8_t> ws(Op::get_workspace_size(args) + 16);  // as the reference testbed does (testbed.h:228-240)
  if (op(args, ws.p) != Status::kSuccess) return false;
  HIP_OK(hipDeviceSynchronize());
  cuasr::reference::host::Srgemm<Add, Mul, T, LA, T, LB, T, LC, T, T> ref;
  ref({m, n, k}, alpha, {A.data(), lda}, {B.data(), ldb}, beta, {C.data(), ldc}, {R.data(), ldc}, Add::Identity);
  D = dD.download();
  return std::memcmp(D.data(), R.data(), D.size() * sizeof(T)) == 0;
}

template <typename Add, typename Mul, typename T> static void testbed_sweep(const char *name) {
  bool ok = true;
  const int ms[2] = {1, 509}, ns[2] = {1, 510}, ks[2] = {1, 23};
  for (int m : ms)
    for (int n : ns)
      for (int k : ks) {
        const T alpha = Mul::Identity, beta = Mul::Annihilator;  // testbed.h:324-325
        ok = ok && testbed_case<Add, Mul, T, ColumnMajor, ColumnMajor, ColumnMajor>(m, n, k, alpha, beta);
        ok = ok && testbed_case<Add, Mul, T, RowMajor, ColumnMajor, RowMajor>(m, n, k, alpha, beta);
        ok = ok && testbed_case<Add, Mul, T, ColumnMajor, RowMajor, RowMajor>(m, n, k, alpha, Mul::Identity);
        ok = ok && testbed_case<Add, Mul, T, RowMajor, RowMajor, ColumnMajor>(m, n, k, alpha, Mul::Identity);
      }
  report(ok, name);
}

// the reference sweep adds split_k_slices = 2, 3, 8 for operators with SplitKSerial (testbed.h:322-338)
template <typename Add, typename Mul, typename T> static void testbed_sweep_serial(const char *name) {
  bool ok = true;
  const int ms[2] = {1, 509}, ns[2] = {1, 510}, ks[2] = {1, 23};
  for (int slices : {1, 2, 3, 8})
    for (int m : ms)
      for (int n : ns)
        for (int k : ks) {
          const T alpha = Mul::Identity;
          ok = ok && testbed_case<Add, Mul, T, ColumnMajor, ColumnMajor, ColumnMajor, true>(m, n, k, alpha, Mul::Annihilator, slices);
          ok = ok && testbed_case<Add, Mul, T, RowMajor, ColumnMajor, RowMajor, true>(m, n, k, alpha, Mul::Identity, slices);
        }
  report(ok, name);
}

// ---- the wider element types through the same operator templates: binary16 throughout (cuasr::half_t), and int8
// operands with int32 results (the element types of the reference's dp4a cores, default_srmma_core_simt.h:747-757)
template <typename Add, typename Mul, typename LA, typename LB, typename LC>
static bool int8_case(int m, int n, int k, int32_t alpha, int32_t beta, int slices = 1) {
  using Op = cuasr::gemm::device::Srgemm<Add, Mul, int8_t, LA, int8_t, LB, int32_t, LC, int32_t>;
  const long long lda = ld_of<LA>(m, k), ldb = ld_of<LB>(k, n), ldc = ld_of<LC>(m, n);
  std::vector<int8_t> A(size_t(m) * k), B(size_t(k) * n);
  std::vector<int32_t> C(size_t(m) * n), D(size_t(m) * n, 0), R(size_t(m) * n, 0);
  fill_int(A, 2019, -128, 127);
  fill_int(B, 2018, -128, 127);
  fill_int(C, 2017, -100000, 100000);
  DeviceBuf<int8_t> dA(A), dB(B);
  DeviceBuf<int32_t> dC(C), dD(D);
  typename Op::Arguments args({m, n, k}, {dA.p, lda}, {dB.p, ldb}, {dC.p, ldc}, {dD.p, ldc}, {alpha, beta}, slices);
  Op op;
  if (Op::can_implement(args) != Status::kSuccess) return false;
  if (op(args, nullptr) != Status::kSuccess) return false;
  HIP_OK(hipDeviceSynchronize());
  cuasr::reference::host::Srgemm<Add, Mul, int8_t, LA, int8_t, LB, int32_t, LC, int32_t, int32_t> ref;
  ref({m, n, k}, alpha, {A.data(), lda}, {B.data(), ldb}, beta, {C.data(), ldc}, {R.data(), ldc}, Add::Identity);
  D = dD.download();
  return std::memcmp(D.data(), R.data(), D.size() * sizeof(int32_t)) == 0;
}

static void wider_element_types() {
  using cuasr::half_t;
  // the conversions of the host-side type, at the places where rounding decides
  bool ok = half_t(1.0f).bits == 0x3c00 && half_t(-2.0f).bits == 0xc000 && half_t(65504.0f).bits == 0x7bff &&
            half_t(65519.9f).bits == 0x7bff && half_t(65520.0f).bits == 0x7c00 && half_t(1.0f + 1.0f / 2048).bits == 0x3c00 &&
            half_t(1.0f + 3.0f / 2048).bits == 0x3c02 && half_t(5.9604645e-8f).bits == 0x0001 && half_t(2.9802322e-8f).bits == 0x0000 &&
            half_t(2.9802326e-8f).bits == 0x0001 && half_t(6.097555e-5f).bits == 0x03ff && half_t(6.1035156e-5f).bits == 0x0400 &&
            half_t(-0.0f).bits == 0x8000 && float(half_t::from_bits(0x0001)) == 5.9604645e-8f && float(half_t::from_bits(0x7bff)) == 65504.0f &&
            float(half_t::from_bits(0xfc00)) == -std::numeric_limits<float>::infinity();
  for (uint32_t b = 0; b < 0x10000 && ok; ++b) {   // every pattern survives the round trip (NaN stays NaN)
    const half_t h = half_t::from_bits(uint16_t(b));
    const float f = float(h);
    ok = (f != f) ? ((half_t(f).bits & 0x7c00) == 0x7c00 && (half_t(f).bits & 0x3ff) != 0) : half_t(f).bits == b;
  }
  report(ok, "cuasr::half_t: conversions round to nearest-even, every pattern survives the round trip");

  ok = true;
  const int ms[2] = {1, 509}, ns[2] = {1, 510}, ks[2] = {1, 23};
  for (int m : ms)
    for (int n : ns)
      for (int k : ks) {
        ok = ok && testbed_case<cuasr::minimum<half_t>, cuasr::plus<half_t>, half_t, ColumnMajor, ColumnMajor, ColumnMajor>(m, n, k, half_t(0), half_t(0));
        ok = ok && testbed_case<cuasr::maximum<half_t>, cuasr::minimum<half_t>, half_t, RowMajor, ColumnMajor, RowMajor>(m, n, k, cuasr::minimum<half_t>::Identity, cuasr::minimum<half_t>::Identity);
        ok = ok && testbed_case<cuasr::plus<half_t>, cuasr::multiplies<half_t>, half_t, ColumnMajor, RowMajor, RowMajor>(m, n, k, half_t(1), half_t(1));
        ok = ok && testbed_case<cuasr::binary_or<half_t>, cuasr::binary_and<half_t>, half_t, RowMajor, RowMajor, ColumnMajor>(m, n, k, half_t(1), half_t(1));
      }
  ok = ok && testbed_case<cuasr::inf::minimum<half_t>, cuasr::plus<half_t>, half_t, RowMajor, ColumnMajor, RowMajor>(256, 512, 96, half_t(0), half_t(0));
  report(ok, "binary16 throughout: min-plus, max-min, plus-times, or-and on the testbed sweep shapes");

  ok = true;
  for (int m : ms)
    for (int n : ns)
      for (int k : ks) {
        ok = ok && int8_case<cuasr::plus<int32_t>, cuasr::multiplies<int32_t>, RowMajor, ColumnMajor, RowMajor>(m, n, k, 1, 0);
        ok = ok && int8_case<cuasr::plus<int32_t>, cuasr::multiplies<int32_t>, ColumnMajor, ColumnMajor, ColumnMajor>(m, n, k, 3, -2);
        ok = ok && int8_case<cuasr::minimum<int32_t>, cuasr::plus<int32_t>, ColumnMajor, RowMajor, RowMajor>(m, n, k, 0, 0);
        ok = ok && int8_case<cuasr::maximum<int32_t>, cuasr::minimum<int32_t>, RowMajor, RowMajor, ColumnMajor>(m, n, k, cuasr::minimum<int32_t>::Identity, cuasr::minimum<int32_t>::Identity);
      }
  ok = ok && int8_case<cuasr::plus<int32_t>, cuasr::multiplies<int32_t>, RowMajor, ColumnMajor, RowMajor>(256, 384, 192, 1, 1);
  report(ok, "int8 operands, int32 results: plus-times, min-plus, max-min on the testbed sweep shapes");

  // half operands with a float accumulator (the reference's spelling of mixed precision): plus-times on the matrix
  // cores, sums in float, D rounded once.  On small integers everything is exact, so the host reference with the same
  // accumulator type must agree bit for bit; a min-plus with that accumulator has no kernel and is refused
  {
    using Add = cuasr::plus<float>;
    using Mul = cuasr::multiplies<float>;
    using Op = cuasr::gemm::device::Srgemm<Add, Mul, half_t, RowMajor, half_t, ColumnMajor, half_t, RowMajor, float>;
    ok = true;
    for (int m : {1, 509, 256})
      for (int k : {1, 23, 192}) {
        const int n = m == 256 ? 384 : 510;
        std::vector<half_t> A(size_t(m) * k), B(size_t(k) * n), C(size_t(m) * n), D(size_t(m) * n), R(size_t(m) * n);
        fill_int(A, 41, -2, 2);
        fill_int(B, 42, -2, 2);
        fill_int(C, 43, -8, 8);
        DeviceBuf<half_t> dA(A), dB(B), dC(C), dD(D);
        Op::Arguments args({m, n, k}, {dA.p, k}, {dB.p, k}, {dC.p, n}, {dD.p, n}, {2.0f, -1.0f});
        Op op;
        ok = ok && Op::can_implement(args) == Status::kSuccess && op(args) == Status::kSuccess;
        HIP_OK(hipDeviceSynchronize());
        cuasr::reference::host::Srgemm<Add, Mul, half_t, RowMajor, half_t, ColumnMajor, half_t, RowMajor, float, float> ref;
        ref({m, n, k}, 2.0f, {A.data(), k}, {B.data(), k}, -1.0f, {C.data(), n}, {R.data(), n}, Add::Identity);
        D = dD.download();
        ok = ok && std::memcmp(D.data(), R.data(), D.size() * sizeof(half_t)) == 0;
      }
    using MinPlus = cuasr::gemm::device::Srgemm<cuasr::minimum<float>, cuasr::plus<float>, half_t, RowMajor, half_t, ColumnMajor, half_t, RowMajor, float>;
    std::vector<half_t> z(64 * 64);
    DeviceBuf<half_t> dz(z);
    MinPlus::Arguments margs({64, 64, 64}, {dz.p, 64}, {dz.p, 64}, {dz.p, 64}, {dz.p, 64}, {0.0f, 0.0f});
    ok = ok && MinPlus::can_implement(margs) == Status::kErrorNotSupported;
    report(ok, "binary16 operands, float accumulator: plus-times on the matrix cores == host reference on small integers");
  }

  // parallel split-K on both: the workspace holds elements of C (2 or 4 bytes each)
  {
    using Add = cuasr::minimum<half_t>;
    using Mul = cuasr::plus<half_t>;
    using SplitK = cuasr::gemm::device::SrgemmSplitKParallel<Add, Mul, half_t, RowMajor, half_t, ColumnMajor, half_t, RowMajor, half_t>;
    using Plain = cuasr::gemm::device::Srgemm<Add, Mul, half_t, RowMajor, half_t, ColumnMajor, half_t, RowMajor, half_t>;
    const int M = 128, N = 96, K = 1000;
    std::vector<half_t> a(size_t(M) * K), b(size_t(K) * N), c(size_t(M) * N);
    fill_unit(a, 21, 0.5, 100.0);
    fill_unit(b, 22, 0.5, 100.0);
    fill_unit(c, 23, 0.5, 100.0);
    DeviceBuf<half_t> da(a), db(b), dc(c), d1(std::vector<half_t>(size_t(M) * N)), d2(std::vector<half_t>(size_t(M) * N));
    ok = true;
    for (int slices : {3, 8}) {
      SplitK::Arguments args({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d1.p, N}, {Mul::Identity, Mul::Identity}, slices);
      const size_t bytes = SplitK::get_workspace_size(args);
      DeviceBuf<uint8_t> ws(bytes);
      SplitK op;
      ok = ok && bytes == sizeof(half_t) * size_t(M) * N * slices;
      ok = ok && op.initialize(args, ws.p) == Status::kSuccess && op() == Status::kSuccess;
      Plain::Arguments pargs({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d2.p, N}, {Mul::Identity, Mul::Identity});
      Plain plain;
      ok = ok && plain(pargs) == Status::kSuccess;
      HIP_OK(hipDeviceSynchronize());
      const std::vector<half_t> x = d1.download(), y = d2.download();
      ok = ok && std::memcmp(x.data(), y.data(), x.size() * sizeof(half_t)) == 0;
    }
    report(ok, "binary16 parallel split-K == non-split");
  }
  {
    using Add = cuasr::plus<int32_t>;
    using Mul = cuasr::multiplies<int32_t>;
    using SplitK = cuasr::gemm::device::SrgemmSplitKParallel<Add, Mul, int8_t, RowMajor, int8_t, ColumnMajor, int32_t, RowMajor, int32_t>;
    using Plain = cuasr::gemm::device::Srgemm<Add, Mul, int8_t, RowMajor, int8_t, ColumnMajor, int32_t, RowMajor, int32_t>;
    const int M = 128, N = 96, K = 1000;
    std::vector<int8_t> a(size_t(M) * K), b(size_t(K) * N);
    std::vector<int32_t> c(size_t(M) * N);
    fill_int(a, 31, -128, 127);
    fill_int(b, 32, -128, 127);
    fill_int(c, 33, -1000, 1000);
    DeviceBuf<int8_t> da(a), db(b);
    DeviceBuf<int32_t> dc(c), d1(std::vector<int32_t>(size_t(M) * N)), d2(std::vector<int32_t>(size_t(M) * N));
    ok = true;
    for (int slices : {3, 8}) {
      SplitK::Arguments args({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d1.p, N}, {2, -3}, slices);
      const size_t bytes = SplitK::get_workspace_size(args);
      DeviceBuf<uint8_t> ws(bytes);
      SplitK op;
      ok = ok && bytes == sizeof(int32_t) * size_t(M) * N * slices;
      ok = ok && op.initialize(args, ws.p) == Status::kSuccess && op() == Status::kSuccess;
      Plain::Arguments pargs({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d2.p, N}, {2, -3});
      Plain plain;
      ok = ok && plain(pargs) == Status::kSuccess;
      HIP_OK(hipDeviceSynchronize());
      ok = ok && d1.download() == d2.download();   // (sums of int32 wrap in any order)
    }
    report(ok, "int8 parallel split-K == non-split");
  }
}

// ---- a user-defined functor, as in examples/01_userdefined_semiring: defined
// by the user, made known to the library by specialising cuasr::op_tag
namespace {
template <typename T, int N = 1> struct my_xor {
  static T constexpr Identity = static_cast<T>(false);
  T operator()(T lhs, T const &rhs) const { lhs ^= rhs; return lhs; }
};
}  // namespace
namespace cuasr {
template <typename T, int N> struct op_tag<my_xor<T, N>> { static int const value = CUASR_AMD_OP_BIT_XOR; };
}

static void example_userdefined_xor_and() {
  using Add = my_xor<int>;
  using Mul = cuasr::binary_and<int>;
  using Op = cuasr::gemm::device::Srgemm<Add, Mul, int, ColumnMajor, int, ColumnMajor, int, ColumnMajor, int>;
  const int M = 256, N = 256, K = 256;
  std::vector<int> A(M * K), B(K * N), C(M * N), R(M * N);
  for (size_t i = 0; i < A.size(); ++i) A[i] = (mix(3090 * 77 + i) % 1000) < 25;  // Bernoulli(0.025), 0/1
  for (size_t i = 0; i < B.size(); ++i) B[i] = (mix(3091 * 77 + i) % 1000) < 25;
  for (size_t i = 0; i < C.size(); ++i) C[i] = (mix(3092 * 77 + i) % 1000) < 25;
  for (int with_c = 0; with_c < 2; ++with_c) {
    DeviceBuf<int> dA(A), dB(B), dC(C);
    const int alpha = Mul::Identity, beta = with_c ? Mul::Identity : Mul::Annihilator;
    typename Op::Arguments args({M, N, K}, {dA.p, M}, {dB.p, K}, {dC.p, M}, {dC.p, M}, {alpha, beta});  // D aliases C
    Op op;
    Status st = op(args, nullptr, nullptr);
    HIP_OK(hipDeviceSynchronize());
    cuasr::reference::host::Srgemm<Add, Mul, int, ColumnMajor, int, ColumnMajor, int, ColumnMajor, int, int> ref;
    ref({M, N, K}, alpha, {A.data(), M}, {B.data(), K}, beta, {C.data(), M}, {R.data(), M}, Add::Identity);
    std::vector<int> D = dC.download();
    report(st == Status::kSuccess && D == R, with_c ? "example01 xor-and (user functor), D = C ^ A.B in place" : "example01 xor-and (user functor)");
  }
}

static void example_minplus_and_known_answer() {
  using Add = cuasr::minimum<float>;
  using Mul = cuasr::plus<float>;
  // the regress vector (test/regress/Srgemm_test.cu:15-62): column-major, D = min(C, A (x) B) in place
  std::vector<float> A = {0.840187728f, 0.911647379f, 0.277774721f, 0.364784479f, 0.394382924f, 0.19755137f, 0.553969979f, 0.513400912f};
  std::vector<float> B = {0.840187728f, 0.911647379f, 0.394382924f, 0.19755137f, 0.729605675f, 0.335222751f, 0.798440039f, 0.768229604f};
  std::vector<float> C = {0.840187728f, 0.911647379f, 0.277774721f, 0.364784479f, 0.394382924f, 0.197551370f, 0.553969979f, 0.513400912f,
                          0.729605675f, 0.335222751f, 0.477397054f, 0.952229738f, 0.798440039f, 0.768229604f, 0.628870904f, 0.916195095f};
  std::vector<float> want = C;
  want[11] = 0.848623633f;
  using OpNN = cuasr::gemm::device::Srgemm<Add, Mul, float, ColumnMajor, float, ColumnMajor, float, ColumnMajor, float>;
  DeviceBuf<float> dA(A), dB(B), dC(C);
  OpNN::Arguments args({4, 4, 2}, {dA.p, 4}, {dB.p, 2}, {dC.p, 4}, {dC.p, 4}, {Mul::Identity, Mul::Identity});
  OpNN op;
  Status st = op(args);
  HIP_OK(hipDeviceSynchronize());
  report(st == Status::kSuccess && dC.download() == want, "regress known-answer 4x4x2 min-plus");

  // example 00: A column-major, B row-major, C/D row-major, 512 cubed, uniform data
  using OpNT = cuasr::gemm::device::Srgemm<Add, Mul, float, ColumnMajor, float, RowMajor, float, RowMajor, float>;
  const int M = 512, N = 512, K = 512;
  std::vector<float> a(M * K), b(K * N), c(M * N), r(M * N);
  fill_unit(a, 1, 0.0, 1.0);
  fill_unit(b, 2, 0.0, 1.0);
  fill_unit(c, 3, 0.0, 1.0);
  DeviceBuf<float> da(a), db(b), dc(c), dd(std::vector<float>(M * N, 0.f));
  const float alpha = Mul::Identity;
  bool ok = true;
  for (float beta : {Mul::Annihilator, Mul::Identity}) {
    OpNT::Arguments g({M, N, K}, {da.p, M}, {db.p, N}, {dc.p, N}, {dd.p, N}, {alpha, beta});
    OpNT o;
    ok = ok && o.initialize(g) == Status::kSuccess && o.run() == Status::kSuccess;
    HIP_OK(hipDeviceSynchronize());
    cuasr::reference::host::Srgemm<Add, Mul, float, ColumnMajor, float, RowMajor, float, RowMajor, float, float> ref;
    ref({M, N, K}, alpha, {a.data(), M}, {b.data(), N}, beta, {c.data(), N}, {r.data(), N}, Add::Identity);
    ok = ok && dd.download() == r;
  }
  report(ok, "example00 min-plus 512^3 (A col, B row, C row), beta = zero and one");

  // update(): same operator object, new output pointer; alpha/beta from device memory
  DeviceBuf<float> dd2(std::vector<float>(M * N, 0.f));
  std::vector<float> ab = {Mul::Identity, Mul::Identity};
  DeviceBuf<float> dab(ab);
  OpNT o;
  OpNT::Arguments g1({M, N, K}, {da.p, M}, {db.p, N}, {dc.p, N}, {dd.p, N}, {alpha, Mul::Identity});
  bool ok2 = o.initialize(g1) == Status::kSuccess;
  OpNT::Arguments g2({M, N, K}, {da.p, M}, {db.p, N}, {dc.p, N}, {dd2.p, N}, {dab.p, dab.p + 1});
  ok2 = ok2 && o.update(g2) == Status::kSuccess && o() == Status::kSuccess;
  HIP_OK(hipDeviceSynchronize());
  report(ok2 && dd2.download() == r, "update() + alpha/beta by device pointer");
}

static void example_splitk() {
  using Add = cuasr::minimum<float>;
  using Mul = cuasr::plus<float>;
  using SplitK = cuasr::gemm::device::SrgemmSplitKParallel<Add, Mul, float, RowMajor, float, ColumnMajor, float, RowMajor, float>;
  using Plain = cuasr::gemm::device::Srgemm<Add, Mul, float, RowMajor, float, ColumnMajor, float, RowMajor, float>;
  const int M = 128, N = 128, K = 4096;  // examples/02_splitk_srgemm/splitk_srgemm.cu:192-199
  std::vector<float> a(size_t(M) * K), b(size_t(K) * N), c(M * N);
  fill_unit(a, 11, 0.5, 1.5);
  fill_unit(b, 12, 0.5, 1.5);
  fill_unit(c, 13, 0.5, 1.5);
  DeviceBuf<float> da(a), db(b), dc(c), d1(std::vector<float>(M * N, 0.f)), d2(std::vector<float>(M * N, 0.f));
  for (int slices : {1, 3, 8, 16}) {
    for (float beta : {Mul::Annihilator, Mul::Identity}) {
      SplitK::Arguments args({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d1.p, N}, {Mul::Identity, beta}, slices);
      const size_t bytes = SplitK::get_workspace_size(args);
      DeviceBuf<uint8_t> ws(bytes);
      SplitK op;
      bool ok = bytes == sizeof(float) * size_t(M) * N * slices;
      ok = ok && op.initialize(args, nullptr) == Status::kErrorWorkspaceNull;
      ok = ok && op.initialize(args, ws.p) == Status::kSuccess && op() == Status::kSuccess;
      Plain::Arguments pargs({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d2.p, N}, {Mul::Identity, beta});
      Plain plain;
      ok = ok && plain(pargs) == Status::kSuccess;
      HIP_OK(hipDeviceSynchronize());
      ok = ok && d1.download() == d2.download();  // the example's own self-check (:270-287)
      char name[96];
      std::snprintf(name, sizeof name, "example02 split-K == non-split, slices=%d beta=%s", slices, beta == Mul::Identity ? "one" : "zero");
      report(ok, name);
    }
  }
  // SplitKSerial = true on the plain operator (device/srgemm.h:83, :218-282): the testbed sizes the workspace
  // with get_workspace_size (testbed.h:228-240); min is idempotent and order-free, so the serial chain
  // equals the unsplit product bit for bit
  using Serial = cuasr::gemm::device::Srgemm<Add, Mul, float, RowMajor, float, ColumnMajor, float, RowMajor, float,
                                             Plain::OperatorClass, Plain::ArchTag, Plain::ThreadblockShape, Plain::WarpShape,
                                             Plain::InstructionShape, Plain::EpilogueOutputOp, Plain::ThreadblockSwizzle,
                                             Plain::kStages, 1, 1, true>;
  static_assert(Serial::kSplitKSerial && !Plain::kSplitKSerial, "kSplitKSerial");
  for (int slices : {1, 2, 3, 8}) {
    Serial::Arguments args({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d1.p, N}, {Mul::Identity, Mul::Identity}, slices);
    const size_t bytes = Serial::get_workspace_size(args);
    DeviceBuf<uint8_t> ws(bytes ? bytes : 16);
    Serial op;
    bool ok = bytes == (slices > 1 ? sizeof(float) * size_t(M) * N * slices : 0);
    ok = ok && Serial::can_implement(args) == Status::kSuccess;
    if (slices > 1) ok = ok && op.initialize(args, nullptr) == Status::kErrorWorkspaceNull;
    ok = ok && op.initialize(args, slices > 1 ? ws.p : nullptr) == Status::kSuccess && op() == Status::kSuccess;
    Plain::Arguments pargs({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d2.p, N}, {Mul::Identity, Mul::Identity});
    Plain plain;
    ok = ok && plain(pargs) == Status::kSuccess;
    HIP_OK(hipDeviceSynchronize());
    ok = ok && d1.download() == d2.download();
    // update(): new output pointer, workspace handed over again (device/srgemm.h:285-300)
    DeviceBuf<float> d3(std::vector<float>(M * N, 0.f));
    Serial::Arguments args3({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d3.p, N}, {Mul::Identity, Mul::Identity}, slices);
    if (slices > 1) ok = ok && op.update(args3, nullptr) == Status::kErrorWorkspaceNull;
    ok = ok && op.update(args3, slices > 1 ? ws.p : nullptr) == Status::kSuccess && op.run() == Status::kSuccess;
    HIP_OK(hipDeviceSynchronize());
    ok = ok && d3.download() == d2.download();
    char name[96];
    std::snprintf(name, sizeof name, "serial split-K (SplitKSerial = true) == non-split, slices=%d", slices);
    report(ok, name);
  }
  // split_k_slices > 1 on the plain operator is an invalid problem (device/srgemm.h:198-200)
  Plain::Arguments bad({M, N, K}, {da.p, K}, {db.p, K}, {dc.p, N}, {d2.p, N}, {Mul::Identity, Mul::Identity}, 4);
  report(Plain::can_implement(bad) == Status::kErrorInvalidProblem && Plain().operator()(bad) == Status::kErrorInvalidProblem,
         "split_k_slices > 1 rejected by Srgemm");
}

// The operator class picks the kernel family: OpClassVectorAlu reproduces the host reference bit for
// bit also for plus-times on non-integer data; the default class may use the matrix cores (rounding
// differs, |d - r| <= 1e-5 * sum|a||b|).
static void operator_classes() {
  using Add = cuasr::plus<float>;
  using Mul = cuasr::multiplies<float>;
  using Exact = cuasr::gemm::device::Srgemm<Add, Mul, float, ColumnMajor, float, ColumnMajor, float, ColumnMajor, float,
                                            cuasr::arch::OpClassVectorAlu>;
  using Auto = cuasr::gemm::device::Srgemm<Add, Mul, float, ColumnMajor, float, ColumnMajor, float, ColumnMajor, float>;
  const int M = 256, N = 128, K = 512;
  std::vector<float> a(size_t(M) * K), b(size_t(K) * N), c(size_t(M) * N), want(size_t(M) * N);
  fill_unit(a, 21, -1.0, 1.0);
  fill_unit(b, 22, -1.0, 1.0);
  fill_unit(c, 23, -1.0, 1.0);
  cuasr::reference::host::Srgemm<Add, Mul, float, ColumnMajor, float, ColumnMajor, float, ColumnMajor, float, float> ref;
  ref({M, N, K}, 1.0f, {a.data(), M}, {b.data(), K}, 1.0f, {c.data(), M}, {want.data(), M}, Add::Identity);
  DeviceBuf<float> da(a), db(b), dc(c), d1(std::vector<float>(size_t(M) * N, 0.f)), d2(std::vector<float>(size_t(M) * N, 0.f));
  Exact::Arguments e({M, N, K}, {da.p, M}, {db.p, K}, {dc.p, M}, {d1.p, M}, {1.0f, 1.0f});
  Auto::Arguments u({M, N, K}, {da.p, M}, {db.p, K}, {dc.p, M}, {d2.p, M}, {1.0f, 1.0f});
  bool ok = Exact()(e) == Status::kSuccess && Auto()(u) == Status::kSuccess;
  HIP_OK(hipDeviceSynchronize());
  report(ok && d1.download() == want, "OpClassVectorAlu plus-times bit-exact vs host reference");
  const std::vector<float> got = d2.download();
  bool close = ok;
  for (size_t i = 0; i < got.size() && close; ++i) close = std::fabs(double(got[i]) - double(want[i])) <= 1e-5 * (K + 1);
  report(close, "default class plus-times within 1e-5 * sum|a||b| of host reference");
}

int main() {
  int devices = 0;
  if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) {
    std::printf("no GPU\n");
    return 77;
  }
  example_minplus_and_known_answer();
  example_userdefined_xor_and();
  example_splitk();
  operator_classes();
  testbed_sweep<cuasr::plus<float>, cuasr::multiplies<float>, float>("testbed plus-multiplies f32");
  testbed_sweep<cuasr::minimum<float>, cuasr::plus<float>, float>("testbed minimum-plus f32");
  testbed_sweep<cuasr::maximum<float>, cuasr::plus<float>, float>("testbed maximum-plus f32");
  testbed_sweep<cuasr::minimum<float>, cuasr::multiplies<float>, float>("testbed minimum-multiplies f32");
  testbed_sweep<cuasr::maximum<float>, cuasr::multiplies<float>, float>("testbed maximum-multiplies f32");
  testbed_sweep<cuasr::minimum<float>, cuasr::maximum<float>, float>("testbed minimum-maximum f32");
  testbed_sweep<cuasr::maximum<float>, cuasr::minimum<float>, float>("testbed maximum-minimum f32");
  testbed_sweep<cuasr::binary_or<float>, cuasr::binary_and<float>, float>("testbed or-and f32");
  testbed_sweep<cuasr::plus<double>, cuasr::multiplies<double>, double>("testbed plus-multiplies f64");
  testbed_sweep<cuasr::minimum<double>, cuasr::plus<double>, double>("testbed minimum-plus f64");
  testbed_sweep<cuasr::maximum<double>, cuasr::plus<double>, double>("testbed maximum-plus f64");
  testbed_sweep<cuasr::minimum<double>, cuasr::multiplies<double>, double>("testbed minimum-multiplies f64");
  testbed_sweep<cuasr::maximum<double>, cuasr::multiplies<double>, double>("testbed maximum-multiplies f64");
  testbed_sweep<cuasr::minimum<double>, cuasr::maximum<double>, double>("testbed minimum-maximum f64");
  testbed_sweep<cuasr::maximum<double>, cuasr::minimum<double>, double>("testbed maximum-minimum f64");
  testbed_sweep<cuasr::binary_or<double>, cuasr::binary_and<double>, double>("testbed or-and f64");
  testbed_sweep_serial<cuasr::plus<float>, cuasr::multiplies<float>, float>("testbed serial split-K plus-multiplies f32");
  testbed_sweep_serial<cuasr::minimum<float>, cuasr::plus<float>, float>("testbed serial split-K minimum-plus f32");
  testbed_sweep_serial<cuasr::maximum<double>, cuasr::plus<double>, double>("testbed serial split-K maximum-plus f64");
  testbed_sweep_serial<cuasr::maximum<double>, cuasr::minimum<double>, double>("testbed serial split-K maximum-minimum f64");
  testbed_sweep_serial<cuasr::binary_or<float>, cuasr::binary_and<float>, float>("testbed serial split-K or-and f32");
  testbed_sweep<cuasr::inf::minimum<float>, cuasr::inf::plus<float>, float>("testbed inf::minimum-plus f32");
  testbed_sweep<cuasr::inf::maximum<double>, cuasr::inf::plus_for_max<double>, double>("testbed inf::maximum-plus f64");
  wider_element_types();
  std::printf("%d checks, %d failed\n", g_run, g_fail);
  return g_fail;
}
