// Two small kernel families with run-time operators:
//   * the naive SRGEMM (one thread per output element) -- runs any operator
//     pair the element type defines, and serves as an on-device cross-check;
//   * the split-K reduction: D = epilogue(add over slices of workspace, C),
//     the second kernel of the parallel split-K
//     (include/cuasr/reduction/kernel/reduce_split_k.h:146-237), and its
//     ordered variant that replays the serial split-K's chain of epilogues.
#include "semiring.h"

namespace cuasr_amd {

// ---------------------------------------------------------------- naive SRGEMM
// TI: the type A and B are stored in (int8 operands are widened to the int32 everything else is in)
template <typename T, typename TI = T>
__global__ __launch_bounds__(256) void naive_srgemm_kernel(Problem p) {
  const int j = blockIdx.x * 16 + (threadIdx.x & 15);
  const int i = blockIdx.y * 16 + (threadIdx.x >> 4);
  const int z = blockIdx.z;
  if (i >= p.m || j >= p.n) return;
  const EpilogueScalars<T> e = resolve_scalars<T>(p, p.mult_op);
  const TI *A = reinterpret_cast<const TI *>(p.A) + (long long)i * p.sa_m;
  const TI *B = reinterpret_cast<const TI *>(p.B) + (long long)j * p.sb_n;
  int k0 = 0, k1 = p.k;
  if (p.workspace) {
    k0 = z * p.k_per_slice;
    k1 = min(p.k, k0 + p.k_per_slice);
  }
  T acc = e.ident;
  for (int kk = k0; kk < k1; ++kk) {
    const T prod = apply_op<T>(p.mult_op, T(A[(long long)kk * p.sa_k]), T(B[(long long)kk * p.sb_k]));
    acc = apply_op<T>(p.add_op, prod, acc);  // host reference order: add(prod, acc)
  }
  if (p.workspace) {
    reinterpret_cast<T *>(p.workspace)[((long long)z * p.m + i) * p.n + j] = acc;
    return;
  }
  T out = apply_op<T>(p.mult_op, e.alpha, acc);
  if (e.source_needed) {
    const T c = reinterpret_cast<const T *>(p.C)[(long long)i * p.ldc + j];
    out = apply_op<T>(p.add_op, out, apply_op<T>(p.mult_op, e.beta, c));
  }
  reinterpret_cast<T *>(p.D)[(long long)i * p.ldd + j] = out;
}

template <typename T, typename TI = T> static hipError_t launch_naive(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  dim3 grid((p.n + 15) / 16, (p.m + 15) / 16, p.workspace ? p.slices : 1);
  launch_kernel((naive_srgemm_kernel<T, TI>), grid, dim3(256), 0, s, p);
  return take_launch_status();
}

launch_fn find_naive(int dtype) {
  switch (dtype) {
    case CUASR_AMD_F32: return launch_naive<float>;
    case CUASR_AMD_F64: return launch_naive<double>;
    case CUASR_AMD_I32: return launch_naive<int32_t>;
    case CUASR_AMD_U32: return launch_naive<uint32_t>;
    case CUASR_AMD_F16: return launch_naive<half_t>;
    case CUASR_AMD_I8: return (launch_naive<int32_t, int8_t>);
    default: return nullptr;
  }
}

// ------------------------------------------------------------ split-K reduction
// One slice's vector of the workspace.  STREAM: a non-temporal load -- the workspace is read once.
// Two regimes, measured on MI355X: an output of a million elements and more is bound by memory
// bandwidth, and there few loads in flight per thread (small kernels, many resident waves) and
// non-temporal loads win (2048^2 x 16 slices: 65.7 us with eight plain loads in flight, 49.1 us
// with one non-temporal load: 6.2 TB/s); a small output is a handful of workgroups bound by
// latency, and there eight loads in flight win (256^2 x 64 slices: 9.2 us against 19.8 us).
template <typename V, bool STREAM> __device__ __forceinline__ V load_slice(const void *at) {
  if constexpr (STREAM) return __builtin_nontemporal_load(reinterpret_cast<const V *>(at));
  else return *reinterpret_cast<const V *>(at);
}

// Each thread owns V consecutive elements of one row.  acc starts at the
// additive identity and folds the slices in ascending order; when the source
// is not needed it is replaced by the identity and the two-operand epilogue is
// still applied (reduce_split_k.h:212-227).
template <typename T, int V, bool VOUT, int U, bool STREAM>
__global__ __launch_bounds__(256) void reduce_splitk_kernel(Problem p) {
  const EpilogueScalars<T> e = resolve_scalars<T>(p, p.mult_op);
  const long long per_row = (p.n + V - 1) / V;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_row * p.m) return;
  const int i = int(idx / per_row);
  const int j = int(idx % per_row) * V;
  const long long slice = (long long)p.m * p.n;
  const T *ws = reinterpret_cast<const T *>(p.workspace) + (long long)i * p.n + j;
  T acc[V];
#pragma unroll
  for (int v = 0; v < V; ++v) acc[v] = e.ident;
  // U slices' loads are issued before the first is folded, so a thread has U memory
  // requests in flight; the fold itself stays in ascending order
  typedef T vec_t __attribute__((ext_vector_type(V)));
  int s = 0;
  for (; s + U <= p.slices; s += U) {
    vec_t w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) w[u] = load_slice<vec_t, STREAM>(ws + (s + u) * slice);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int v = 0; v < V; ++v) acc[v] = apply_op<T>(p.add_op, acc[v], w[u][v]);
  }
  for (; s < p.slices; ++s) {
    const vec_t w = load_slice<vec_t, STREAM>(ws + s * slice);
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = apply_op<T>(p.add_op, acc[v], w[v]);
  }
  const T *C = reinterpret_cast<const T *>(p.C);
  T *D = reinterpret_cast<T *>(p.D);
  T out[V];
#pragma unroll
  for (int v = 0; v < V; ++v) {
    T src = e.ident;
    if (e.source_needed && j + v < p.n) src = C[(long long)i * p.ldc + j + v];
    const T lhs = apply_op<T>(p.mult_op, e.alpha, acc[v]);
    out[v] = apply_op<T>(p.add_op, lhs, apply_op<T>(p.mult_op, e.beta, src));
  }
  T *dst = D + (long long)i * p.ldd + j;
  if (V > 1 && VOUT) {  // one 16-byte store (the host checked alignment and that n is a multiple of V)
    vec_t o;
#pragma unroll
    for (int v = 0; v < V; ++v) o[v] = out[v];
    *reinterpret_cast<vec_t *>(dst) = o;
  } else {
#pragma unroll
    for (int v = 0; v < V; ++v)
      if (j + v < p.n) dst[v] = out[v];
  }
}

// The ordered fold of the serial split-K.  In the reference the workgroups of one
// output tile take turns, slice 0 first: slice 0 writes
// D = add(mult(alpha, acc_0), mult(beta, C)) (or mult(alpha, acc_0) when the source
// is not needed), every later slice z reads D back as its source with beta replaced
// by the multiplicative identity and writes D = add(mult(alpha, acc_z), mult(one, D))
// (include/cuasr/gemm/kernel/srgemm.h:249-320,
// epilogue/thread/semiring_linear_combination.h:119-134).  Here the slices' raw
// accumulators are in the workspace and one thread replays that chain for its
// elements in registers: same operands, same order, one write of D.
template <typename T, int V, bool VOUT, int U, bool STREAM>
__global__ __launch_bounds__(256) void reduce_serial_kernel(Problem p) {
  const EpilogueScalars<T> e = resolve_scalars<T>(p, p.mult_op);
  const T one = scalar_as<T>(p.mult_identity);
  // "source needed" as a later slice's epilogue evaluates it, with beta = one
  const bool chain = e.ident != apply_op<T>(p.mult_op, one, one);
  const long long per_row = (p.n + V - 1) / V;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= per_row * p.m) return;
  const int i = int(idx / per_row);
  const int j = int(idx % per_row) * V;
  const long long slice = (long long)p.m * p.n;
  const T *ws = reinterpret_cast<const T *>(p.workspace) + (long long)i * p.n + j;
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const T *C = reinterpret_cast<const T *>(p.C);
  T out[V];
  {
    const vec_t w = load_slice<vec_t, STREAM>(ws);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      out[v] = apply_op<T>(p.mult_op, e.alpha, w[v]);
      if (e.source_needed && j + v < p.n)
        out[v] = apply_op<T>(p.add_op, out[v], apply_op<T>(p.mult_op, e.beta, C[(long long)i * p.ldc + j + v]));
    }
  }
  auto step = [&](const vec_t &w) {
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const T lhs = apply_op<T>(p.mult_op, e.alpha, w[v]);
      out[v] = chain ? apply_op<T>(p.add_op, lhs, apply_op<T>(p.mult_op, one, out[v])) : lhs;
    }
  };
  int s = 1;  // U loads in flight per thread, as in the parallel reduction
  for (; s + U <= p.slices; s += U) {
    vec_t w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) w[u] = load_slice<vec_t, STREAM>(ws + (s + u) * slice);
#pragma unroll
    for (int u = 0; u < U; ++u) step(w[u]);
  }
  for (; s < p.slices; ++s) step(load_slice<vec_t, STREAM>(ws + s * slice));
  T *dst = reinterpret_cast<T *>(p.D) + (long long)i * p.ldd + j;
  if (V > 1 && VOUT) {
    vec_t o;
#pragma unroll
    for (int v = 0; v < V; ++v) o[v] = out[v];
    *reinterpret_cast<vec_t *>(dst) = o;
  } else {
#pragma unroll
    for (int v = 0; v < V; ++v)
      if (j + v < p.n) dst[v] = out[v];
  }
}

template <typename T, bool SERIAL, int V, bool VOUT> static void launch_one(const Problem &p, dim3 grid, hipStream_t s) {
  constexpr int U = V > 1 ? 1 : 8;      // the 16-byte path is the large-output one
  constexpr bool STREAM = V > 1;
  // (the serial form's chain of run-time operators, not memory, bounds it: 65 - 67 us at any depth)
  if (SERIAL) launch_kernel((reduce_serial_kernel<T, V, VOUT, (V > 1 ? 2 : 8), STREAM>), grid, dim3(256), 0, s, p);
  else launch_kernel((reduce_splitk_kernel<T, V, VOUT, U, STREAM>), grid, dim3(256), 0, s, p);
}

template <typename T, bool SERIAL> static hipError_t launch_reduce(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  constexpr int V = 16 / sizeof(T);
  const bool vec = (p.n % V == 0) && (reinterpret_cast<uintptr_t>(p.workspace) % 16 == 0);
  // small outputs: one element per thread gives V times as many workgroups to spread over the chip
  const bool small = (long long)p.m * p.n < 256LL * 1024 * V;
  if (vec && !small) {
    const long long work = (long long)p.m * (p.n / V);
    const dim3 grid((unsigned)((work + 255) / 256));
    if (reinterpret_cast<uintptr_t>(p.D) % 16 == 0 && p.ldd % V == 0) launch_one<T, SERIAL, V, true>(p, grid, s);
    else launch_one<T, SERIAL, V, false>(p, grid, s);
  } else {
    const long long work = (long long)p.m * p.n;
    launch_one<T, SERIAL, 1, false>(p, dim3((unsigned)((work + 255) / 256)), s);
  }
  return take_launch_status();
}

// ------------------------------------------------------------ source term for the stream-K tiles
// D <- mult(beta, C) where the source is needed, else the additive identity, on the output tiles (bm x bn) from
// `first` on in the stream-K tile order: what the workgroups that share those tiles fold their ranges of k into
// (the epilogue's add then has nothing left to do).  One workgroup per tile.  D may be C.
template <typename T> __global__ __launch_bounds__(256) void prepare_fold_kernel(Problem p, int bm, int bn, long long first) {
  const EpilogueScalars<T> e = resolve_scalars<T>(p, p.mult_op);
  const int tiles_m = (p.m + bm - 1) / bm, tiles_n = (p.n + bn - 1) / bn;
  int tm, tn;
  streamk_tile_coords(first + blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * bm, n0 = tn * bn;
  for (int idx = threadIdx.x; idx < bm * bn; idx += 256) {
    const int row = m0 + idx / bn, col = n0 + idx % bn;
    if (row < p.m && col < p.n) {
      T v = e.ident;
      if (e.source_needed) v = apply_op<T>(p.mult_op, e.beta, reinterpret_cast<const T *>(p.C)[(long long)row * p.ldc + col]);
      reinterpret_cast<T *>(p.D)[(long long)row * p.ldd + col] = v;
    }
  }
}

template <typename T> static hipError_t launch_prepare_fold(const Problem &p, int bm, int bn, long long first, hipStream_t s) {
  const long long tiles = (long long)((p.m + bm - 1) / bm) * ((p.n + bn - 1) / bn);
  if (tiles <= first) return hipSuccess;
  launch_kernel(prepare_fold_kernel<T>, dim3((unsigned)(tiles - first)), dim3(256), 0, s, p, bm, bn, first);
  return take_launch_status();
}

prepare_fold_fn find_prepare_fold(int dtype) {
  switch (dtype) {
    case CUASR_AMD_F32: return launch_prepare_fold<float>;
    case CUASR_AMD_I32: return launch_prepare_fold<int32_t>;
    case CUASR_AMD_U32: return launch_prepare_fold<uint32_t>;
    default: return nullptr;
  }
}

launch_fn find_reduce(int dtype) {
  switch (dtype) {
    case CUASR_AMD_F32: return launch_reduce<float, false>;
    case CUASR_AMD_F64: return launch_reduce<double, false>;
    case CUASR_AMD_I32: return launch_reduce<int32_t, false>;
    case CUASR_AMD_U32: return launch_reduce<uint32_t, false>;
    case CUASR_AMD_F16: return launch_reduce<half_t, false>;
    case CUASR_AMD_I8: return launch_reduce<int32_t, false>;   // (the partial products are int32)
    default: return nullptr;
  }
}

launch_fn find_reduce_serial(int dtype) {
  switch (dtype) {
    case CUASR_AMD_F32: return launch_reduce<float, true>;
    case CUASR_AMD_F64: return launch_reduce<double, true>;
    case CUASR_AMD_I32: return launch_reduce<int32_t, true>;
    case CUASR_AMD_U32: return launch_reduce<uint32_t, true>;
    case CUASR_AMD_F16: return launch_reduce<half_t, true>;
    case CUASR_AMD_I8: return launch_reduce<int32_t, true>;
    default: return nullptr;
  }
}

}  // namespace cuasr_amd
