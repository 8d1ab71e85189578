// Call sites spelled the way programs written against cuASR spell them -- cutlass:: names for layouts, operator
// class, architecture tag, tile shapes, swizzle, status and the workspace buffer; brace-initialised Arguments;
// a user-defined addition functor with the three cutlass::Array overloads -- compiled against this library's
// headers with nothing changed but the stream type and the memory calls (HIP's).  The three shapes follow
//   examples/00_minplus_srgemm/minplus_srgemm.cu:9-65           (default configuration, nine template arguments)
//   examples/01_userdefined_semiring/userdefined_semiring.cu:56-177  (every tuning argument spelled out, user functor)
//   examples/02_splitk_srgemm/splitk_srgemm.cu:17-86            (SrgemmSplitKParallel, workspace from get_workspace_size)
// of the reference, and each result is compared bit for bit with the host reference SRGEMM, as the examples do
// (minplus_srgemm.cu:150-190, userdefined_semiring.cu:253-273, splitk_srgemm.cu:270-287).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "cuasr/functional.h"
#include "cuasr/gemm/device/default_srgemm_configuration.h"
#include "cuasr/gemm/device/srgemm.h"
#include "cuasr/gemm/device/srgemm_splitk_parallel.h"
#include "cuasr/reference/srgemm/host_srgemm.h"

static int g_run = 0, g_fail = 0;
static void report(bool ok, const char *what) {
  ++g_run;
  if (!ok) ++g_fail;
  std::printf("%s %s\n", ok ? "PASS" : "FAIL", what);
}

template <typename T> struct Device {
  T *p = nullptr;
  size_t n;
  explicit Device(std::vector<T> const &h) : n(h.size()) {
    if (hipMalloc(&p, n * sizeof(T)) != hipSuccess || hipMemcpy(p, h.data(), n * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) std::exit(2);
  }
  ~Device() { (void)hipFree(p); }
  std::vector<T> host() const {
    std::vector<T> h(n);
    if (hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost) != hipSuccess) std::exit(2);
    return h;
  }
};

// ---- tropical SRGEMM with the default configuration -----------------------------------------------------
static int tropical_nt_n(int M, int N, int K, float const *A, int lda, float const *B, int ldb, float *C, int ldc, float *D,
                         bool fold_c_in, hipStream_t stream = nullptr) {
  using OperatorClass = cutlass::arch::OpClassSimt;
  using SmArch = cutlass::arch::Sm50;
  using AdditionOp = cuasr::minimum<float>;
  using MultiplicationOp = cuasr::plus<float>;
  using Config = typename cuasr::gemm::device::DefaultSemiRingConfiguration<float, float, float, float, OperatorClass, AdditionOp,
                                                                            MultiplicationOp, SmArch>;
  static_assert(Config::kStages >= 2, "the configuration type is complete");
  using ColumnMajor = cutlass::layout::ColumnMajor;
  using RowMajor = cutlass::layout::RowMajor;
  using Tropical = cuasr::gemm::device::Srgemm<AdditionOp, MultiplicationOp, float, ColumnMajor, float, RowMajor, float, ColumnMajor, float>;
  float alpha = MultiplicationOp::Identity;
  float beta = fold_c_in ? MultiplicationOp::Identity : MultiplicationOp::Annihilator;
  Tropical::Arguments args({M, N, K}, {A, lda}, {B, ldb}, {C, ldc}, {D, ldc}, {alpha, beta});
  Tropical op;
  cutlass::Status status = op(args, nullptr, stream);
  return static_cast<int>(status);
}

// ---- a semiring of the caller's own: xor as addition, with the Array forms a cuASR functor carries -----
namespace {
template <typename T, int N = 1> struct galois_add {
  static T constexpr Identity = static_cast<T>(false);
  __host__ __device__ T operator()(T lhs, T const &rhs) const {
    lhs ^= rhs;
    return lhs;
  }
  __host__ __device__ cutlass::Array<T, N> operator()(cutlass::Array<T, N> const &lhs, cutlass::Array<T, N> const &rhs) const {
    cutlass::Array<T, N> result;
    for (int i = 0; i < N; ++i) result[i] = this->operator()(lhs[i], rhs[i]);
    return result;
  }
  __host__ __device__ cutlass::Array<T, N> operator()(cutlass::Array<T, N> const &lhs, T const &scalar) const {
    cutlass::Array<T, N> result;
    for (int i = 0; i < N; ++i) result[i] = this->operator()(lhs[i], scalar);
    return result;
  }
  __host__ __device__ cutlass::Array<T, N> operator()(T const &scalar, cutlass::Array<T, N> const &rhs) const {
    cutlass::Array<T, N> result;
    for (int i = 0; i < N; ++i) result[i] = this->operator()(scalar, rhs[i]);
    return result;
  }
};
}  // namespace

static int galois_nnn(int M, int N, int K, int const *A, int lda, int const *B, int ldb, int *C, int ldc, int *D, bool fold_c_in,
                      hipStream_t stream = nullptr) {
  using OperatorClass = cutlass::arch::OpClassSimt;
  using SmArch = cutlass::arch::Sm50;
  using AdditionOp = galois_add<int>;
  using MultiplicationOp = cuasr::binary_and<int>;
  using EpilogueOutputOp = cuasr::epilogue::thread::SemiringLinearCombination<AdditionOp, MultiplicationOp, int, 1>;
  static int constexpr AlignmentA = 1;
  static int constexpr AlignmentB = 1;
  using ThreadblockShape = cutlass::gemm::GemmShape<64, 128, 8>;
  using WarpShape = cutlass::gemm::GemmShape<16, 64, 8>;
  using InstructionShape = cutlass::gemm::GemmShape<1, 1, 1>;
  using ThreadblockSwizzle = typename cutlass::gemm::threadblock::GemmIdentityThreadblockSwizzle<>;
  static int constexpr Stages = 2;
  using RowMajor = cutlass::layout::RowMajor;
  using Galois = cuasr::gemm::device::Srgemm<AdditionOp, MultiplicationOp, int, RowMajor, int, RowMajor, int, RowMajor, int, OperatorClass,
                                             SmArch, ThreadblockShape, WarpShape, InstructionShape, EpilogueOutputOp, ThreadblockSwizzle,
                                             Stages, AlignmentA, AlignmentB, false>;
  int alpha = MultiplicationOp::Identity;
  int beta = fold_c_in ? MultiplicationOp::Identity : MultiplicationOp::Annihilator;
  Galois::Arguments args({M, N, K}, {A, lda}, {B, ldb}, {C, ldc}, {D, ldc}, {alpha, beta});
  Galois op;
  cutlass::Status status = op(args, nullptr, stream);
  return static_cast<int>(status);
}

// ---- parallel split-K with a workspace sized by the operator ------------------------------------------
static int tropical_splitk_tn_t(int M, int N, int K, float const *A, int lda, float const *B, int ldb, float *C, int ldc, float *D,
                                bool fold_c_in, int split_k_slices, hipStream_t stream = nullptr) {
  using AdditionOp = cuasr::minimum<float>;
  using MultiplicationOp = cuasr::plus<float>;
  using ColumnMajor = cutlass::layout::ColumnMajor;
  using RowMajor = cutlass::layout::RowMajor;
  using SplitK = cuasr::gemm::device::SrgemmSplitKParallel<AdditionOp, MultiplicationOp, float, RowMajor, float, ColumnMajor, float, RowMajor, float>;
  float alpha = MultiplicationOp::Identity;
  float beta = fold_c_in ? MultiplicationOp::Identity : MultiplicationOp::Annihilator;
  SplitK::Arguments args({M, N, K}, {A, lda}, {B, ldb}, {C, ldc}, {D, ldc}, {alpha, beta}, split_k_slices);
  size_t workspace_size = SplitK::get_workspace_size(args);
  cutlass::device_memory::allocation<uint8_t> workspace(workspace_size);
  SplitK op;
  cutlass::Status status = op.initialize(args, workspace.get());
  if (status != cutlass::Status::kSuccess) return static_cast<int>(status);
  status = op(stream);
  return static_cast<int>(status);
}

int main() {
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count == 0) {
    std::printf("no GPU\n");
    return 1;
  }
  {
    const int M = 384, N = 256, K = 300;
    std::vector<float> A(size_t(M) * K), B(size_t(K) * N), C(size_t(M) * N), R(C.size());
    std::mt19937_64 rng(7);
    std::uniform_real_distribution<float> dist(0.5f, 1.5f);
    for (auto &v : A) v = dist(rng);
    for (auto &v : B) v = dist(rng);
    for (auto &v : C) v = dist(rng);
    for (bool fold : {true, false}) {
      Device<float> dA(A), dB(B), dC(C);
      const int rc = tropical_nt_n(M, N, K, dA.p, M, dB.p, N, dC.p, M, dC.p, fold);   // D aliases C, as in the example
      if (hipDeviceSynchronize() != hipSuccess) return 2;
      using Add = cuasr::minimum<float>;
      using Mul = cuasr::plus<float>;
      cuasr::reference::host::Srgemm<Add, Mul, float, cutlass::layout::ColumnMajor, float, cutlass::layout::RowMajor, float,
                                     cutlass::layout::ColumnMajor, float, float> ref;
      ref({M, N, K}, Mul::Identity, {A.data(), M}, {B.data(), N}, fold ? Mul::Identity : Mul::Annihilator, {C.data(), M}, {R.data(), M}, Add::Identity);
      const std::vector<float> D = dC.host();
      report(rc == 0 && std::memcmp(D.data(), R.data(), D.size() * 4) == 0,
             fold ? "min-plus, default configuration, D = min(C, A (x) B) in place" : "min-plus, default configuration, beta = annihilator");
    }
  }
  {
    const int M = 512, N = 512, K = 512;
    std::vector<int> A(size_t(M) * K), B(size_t(K) * N), C(size_t(M) * N), R(C.size());
    std::mt19937_64 rng(3090);
    std::bernoulli_distribution dist(0.025);
    for (auto &v : A) v = int(dist(rng));
    for (auto &v : B) v = int(dist(rng));
    for (auto &v : C) v = int(dist(rng));
    Device<int> dA(A), dB(B), dC(C);
    const int rc = galois_nnn(M, N, K, dA.p, K, dB.p, N, dC.p, N, dC.p, true);
    if (hipDeviceSynchronize() != hipSuccess) return 2;
    using Add = galois_add<int>;
    using Mul = cuasr::binary_and<int>;
    using RowMajor = cutlass::layout::RowMajor;
    cuasr::reference::host::Srgemm<Add, Mul, int, RowMajor, int, RowMajor, int, RowMajor, int, int> ref;
    ref({M, N, K}, Mul::Identity, {A.data(), K}, {B.data(), N}, Mul::Identity, {C.data(), N}, {R.data(), N}, Add::Identity);
    const std::vector<int> D = dC.host();
    report(rc == 0 && std::memcmp(D.data(), R.data(), D.size() * 4) == 0, "GF(2) xor-and with a user-defined addition, every tuning argument spelled out");
    cutlass::Array<int, 4> x{}, y{};
    for (int i = 0; i < 4; ++i) {
      x[i] = i;
      y[i] = 3;
    }
    const cutlass::Array<int, 4> z = galois_add<int, 4>()(x, y), w = cuasr::plus<int, 4>()(x, 10), u = cuasr::minimum<int, 4>()(2, x);
    report(z[0] == 3 && z[1] == 2 && z[3] == 0 && w[2] == 12 && u[0] == 0 && u[3] == 2, "Array forms: user functor and library functors, array / scalar operands");
  }
  {
    const int M = 128, N = 128, K = 4096;
    std::vector<float> A(size_t(M) * K), B(size_t(K) * N), C(size_t(M) * N), R(C.size());
    std::mt19937_64 rng(11);
    std::uniform_real_distribution<float> dist(0.5f, 1.5f);
    for (auto &v : A) v = dist(rng);
    for (auto &v : B) v = dist(rng);
    for (auto &v : C) v = dist(rng);
    using Add = cuasr::minimum<float>;
    using Mul = cuasr::plus<float>;
    cuasr::reference::host::Srgemm<Add, Mul, float, cutlass::layout::RowMajor, float, cutlass::layout::ColumnMajor, float,
                                   cutlass::layout::RowMajor, float, float> ref;
    ref({M, N, K}, Mul::Identity, {A.data(), K}, {B.data(), K}, Mul::Identity, {C.data(), N}, {R.data(), N}, Add::Identity);
    for (int slices : {1, 8, 13}) {
      Device<float> dA(A), dB(B), dC(C);
      const int rc = tropical_splitk_tn_t(M, N, K, dA.p, K, dB.p, K, dC.p, N, dC.p, true, slices);
      if (hipDeviceSynchronize() != hipSuccess) return 2;
      const std::vector<float> D = dC.host();
      char name[96];
      std::snprintf(name, sizeof name, "parallel split-K min-plus 128x128x4096, %d slices == the unsplit host result", slices);
      report(rc == 0 && std::memcmp(D.data(), R.data(), D.size() * 4) == 0, name);
    }
  }
  std::printf("%d checks, %d failed\n", g_run, g_fail);
  return g_fail ? 1 : 0;
}
