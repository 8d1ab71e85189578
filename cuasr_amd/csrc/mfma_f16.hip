// Plus-times on binary16 operands with float accumulation, on the matrix cores -- by request only.
//
// The library's own binary16 plus-times (half_tile.h) rounds every product and every partial sum to binary16, as
// the reference's templates would with a half type for every element (arch/srmma.h:65-92 in ElementC), and is
// bit-identical to the CPU oracle.  This kernel is the other thing a caller may mean by a half-precision GEMM, the
// reference's ElementAccumulator = float: products of binary16 values are exact in float, the sums run in float on
// v_mfma_f32_32x32x16_f16, and only D = alpha * acc + beta * C is rounded to binary16, once.  More accurate than the
// oracle's running binary16 sum and an order of magnitude faster than the vector ALU, but not bit-identical to it:
// it runs only when the descriptor names the matrix-core family, never by the library's own choice.
//
// Same shape as the int8 kernel (mfma_i8.hip): 256 threads (2 x 2 waves), tile 128 x 128 x 64, a wave holds 2 x 2
// blocks of 32 x 32 (64 accumulator registers), two workgroups per compute unit; every lane supplies 8 consecutive k
// of one row (column) per instruction; LDS holds both panels k-contiguous, [x][64 k + 8 of padding], two stages;
// the loads of k-tile t + 2 are issued before tile t is worked on.  An operand whose rows (columns) are contiguous in
// memory is transposed in registers on its way to LDS: two 16-byte loads of 8 x at k and k + 1 become 8 words of
// (x; k, k + 1).
#include "semiring.h"

namespace cuasr_amd {

// the hand-scheduled form for whole 256 x 256 tiles of k-contiguous operands (mfma_direct_narrow.hip)
bool mfma_narrow_f16_can_run(const Problem &p, int units);
hipError_t launch_mfma_narrow_f16(const Problem &p, hipStream_t s);

namespace mfma_f16 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef half_t v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 64, THREADS = 256, PITCH = BK + 8;  // (elements; a row of a panel is 144 bytes)
constexpr int KCH = BK / 8;  // 16-byte chunks along k

struct Smem {
  half_t a[2][BM][PITCH];
  half_t b[2][BN][PITCH];
};

// One operand's share of a k-tile (X x, BK k) on its way from memory to LDS.
//   KC (k contiguous in memory): chunks of 8 k of one x, written as they are.
//   otherwise (x contiguous):    units of 8 x by 2 k; two 16-byte loads, transposed in registers.
// GUARD: elements beyond the extents read as zero (a zero factor adds nothing to a sum of products).
template <int X, bool KC, bool GUARD> struct Stager {
  static constexpr int CHUNKS = KCH * X / THREADS;          // KC: 16-byte chunks per thread
  static constexpr int UNITS = (X / 8) * (BK / 2) / THREADS;  // otherwise: units per thread
  static_assert(KCH * X % THREADS == 0 && (X / 8) * (BK / 2) % THREADS == 0, "a panel splits evenly over the threads");
  v4i r[KC ? CHUNKS : 2 * UNITS];
  // unit u -> (x, k) of its first element.  XB neighbouring lanes take neighbouring blocks of 8 x at one pair of k,
  // the next lanes the next pairs of k: the lanes of one LDS store then write XB rows that are 8 apart (8 rows of 144
  // bytes = 32 banks) at 64 / XB consecutive words each.
#ifndef CUASR_F16_XB
#define CUASR_F16_XB 2
#endif
  static constexpr int XB = CUASR_F16_XB;
  static_assert((X / 8) % XB == 0, "blocks of x split evenly");
  static __device__ __forceinline__ void where(int u, int &x, int &k) {
    const int lo = u % XB, kp = (u / XB) % (BK / 2), hi = u / (XB * (BK / 2));
    x = (hi * XB + lo) * 8;
    k = kp * 2;
  }

  static __device__ __forceinline__ v4i fetch(const half_t *src, int first, int limit, bool live) {
    // 8 consecutive elements; element e is number first + e of a run that ends at `limit`
    if constexpr (!GUARD) {
      return *reinterpret_cast<const v4i *>(src);
    } else {
      v4i v = {0, 0, 0, 0};
      typedef int loose4 __attribute__((ext_vector_type(4), aligned(2)));  // (a vector load may start at any element)
      if (live && first + 8 <= limit) {
        v = *reinterpret_cast<const loose4 *>(src);
      } else if (live) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int bits = (first + e < limit) ? (int)__builtin_bit_cast(unsigned short, src[e]) : 0;
          v[e / 2] |= bits << (16 * (e % 2));
        }
      }
      return v;
    }
  }

  __device__ __forceinline__ void load(const half_t *base, long long sx, long long sk, int x0, int k0, int xn, int kn) {
    if constexpr (KC) {
#pragma unroll
      for (int q = 0; q < CHUNKS; ++q) {
        const int c = threadIdx.x + q * THREADS, k = (c % KCH) * 8, x = c / KCH;
        r[q] = fetch(base + (long long)(x0 + x) * sx + (k0 + k), k0 + k, kn, x0 + x < xn);
      }
    } else {
#pragma unroll
      for (int q = 0; q < UNITS; ++q) {
        const int u = threadIdx.x + q * THREADS;
        int x, k;
        where(u, x, k);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
          r[2 * q + kk] = fetch(base + (x0 + x) + (long long)(k0 + k + kk) * sk, x0 + x, xn, k0 + k + kk < kn);
      }
    }
  }

  __device__ __forceinline__ void store(half_t (*panel)[PITCH]) const {
    if constexpr (KC) {
#pragma unroll
      for (int q = 0; q < CHUNKS; ++q) {
        const int c = threadIdx.x + q * THREADS, k = (c % KCH) * 8, x = c / KCH;
        *reinterpret_cast<v4i *>(&panel[x][k]) = r[q];
      }
    } else {
#pragma unroll
      for (int q = 0; q < UNITS; ++q) {
        const int u = threadIdx.x + q * THREADS;
        int x, k;
        where(u, x, k);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          // word d of the two loads holds x = 2d, 2d + 1 at k and at k + 1: a 2 x 2 transpose of 16-bit elements
          const unsigned at_k = r[2 * q + 0][d], at_k1 = r[2 * q + 1][d];
          *reinterpret_cast<unsigned *>(&panel[x + 2 * d + 0][k]) = __builtin_amdgcn_perm(at_k1, at_k, 0x05040100);
          *reinterpret_cast<unsigned *>(&panel[x + 2 * d + 1][k]) = __builtin_amdgcn_perm(at_k1, at_k, 0x07060302);
        }
      }
    }
  }
};

template <bool A_KC, bool B_KC, bool GUARD>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void mfma_f16_kernel(Problem p) {
  __shared__ __attribute__((aligned(16))) Smem sm;
  select_batch<half_t>(p);
  const int tiles_n = (p.n + BN - 1) / BN;
  const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, half = lane >> 5;
  const half_t *A = reinterpret_cast<const half_t *>(p.A), *B = reinterpret_cast<const half_t *>(p.B);
  const int kb = 0, ke = p.k;  // (no split-K form: partial sums would have to leave as binary16)

  v16f acc[2][2];
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[bi][bj][e] = 0.0f;

  Stager<BM, A_KC, GUARD> sa[2];
  Stager<BN, B_KC, GUARD> sb[2];
  const int tiles_k = ke > kb ? (ke - kb + BK - 1) / BK : 0;
  if (tiles_k > 0) {
    sa[1].load(A, p.sa_m, p.sa_k, m0, kb, p.m, ke);
    sb[1].load(B, p.sb_n, p.sb_k, n0, kb, p.n, ke);
    if (tiles_k > 1) {
      sa[0].load(A, p.sa_m, p.sa_k, m0, kb + BK, p.m, ke);
      sb[0].load(B, p.sb_n, p.sb_k, n0, kb + BK, p.n, ke);
    }
    sa[1].store(sm.a[0]);
    sb[1].store(sm.b[0]);
  }
  __syncthreads();
  // one k-tile: `la`, `lb` take the loads of tile t + 2; `ha`, `hb` hold tile t + 1, which goes to LDS afterwards
  auto tile = [&](int t, auto &la, auto &lb, const auto &ha, const auto &hb) {
    const int s = t & 1, k0 = kb + t * BK;
    if (t + 2 < tiles_k) {
      la.load(A, p.sa_m, p.sa_k, m0, k0 + 2 * BK, p.m, ke);
      lb.load(B, p.sb_n, p.sb_k, n0, k0 + 2 * BK, p.n, ke);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      v8h a[2], b[2];
#pragma unroll
      for (int bi = 0; bi < 2; ++bi) a[bi] = *reinterpret_cast<const v8h *>(&sm.a[s][wm * 64 + bi * 32 + l32][ks * 16 + half * 8]);
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) b[bj] = *reinterpret_cast<const v8h *>(&sm.b[s][wn * 64 + bj * 32 + l32][ks * 16 + half * 8]);
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[bi], b[bj], acc[bi][bj], 0, 0, 0);
    }
    if (t + 1 < tiles_k) {
      ha.store(sm.a[s ^ 1]);
      hb.store(sm.b[s ^ 1]);
    }
    __syncthreads();
  };
  for (int t = 0; t < tiles_k; t += 2) {
    tile(t, sa[1], sb[1], sa[0], sb[0]);
    if (t + 1 < tiles_k) tile(t + 1, sa[0], sb[0], sa[1], sb[1]);
  }

  // ---- epilogue.  Register e of lane l in block (bi, bj): row 8*(e/4) + 4*(l/32) + e%4, column l%32.
  // D = alpha * acc + beta * C in float, rounded to binary16 once.
  const EpilogueScalars<half_t> sc = resolve_scalars<half_t>(p, kMultiplies);
  const float alpha = float(sc.alpha), beta = float(sc.beta);
  const half_t *C = reinterpret_cast<const half_t *>(p.C);
  half_t *D = reinterpret_cast<half_t *>(p.D);
  // A store instruction writes 64 consecutive bytes of two rows; the two blocks of a block row are stored register by
  // register, so that consecutive instructions write consecutive pieces of the same rows, and a block row's source
  // elements are requested together, before any of its results is stored (D may be C, so the compiler cannot move a
  // load of C above a store to D by itself)
#pragma unroll
  for (int bi = 0; bi < 2; ++bi) {
    auto row_of = [&](int e) { return m0 + wm * 64 + bi * 32 + 8 * (e / 4) + 4 * half + (e % 4); };
    auto inside = [&](int row, int col) { return !GUARD || ((unsigned)row < (unsigned)p.m && (unsigned)col < (unsigned)p.n); };
    half_t src[16][2];
    if (sc.source_needed) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) {
          const int row = row_of(e), col = n0 + wn * 64 + bj * 32 + l32;
          src[e][bj] = inside(row, col) ? C[(long long)row * p.ldc + col] : half_t(0);
        }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) {
        const int row = row_of(e), col = n0 + wn * 64 + bj * 32 + l32;
        if (!inside(row, col)) continue;
        float out = alpha * acc[bi][bj][e];
        if (sc.source_needed) out += beta * float(src[e][bj]);
        D[(long long)row * p.ldd + col] = half_t(out);
      }
  }
}

// whole tiles of 16-byte aligned operands: the unguarded kernel
static bool exact(const Problem &p, bool a_kc, bool b_kc) {
  auto al16 = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  if (p.m % BM || p.n % BN || p.k % BK || p.k == 0) return false;
  if ((a_kc ? p.sa_m : p.sa_k) % 8 || (b_kc ? p.sb_n : p.sb_k) % 8) return false;
  if (!al16(p.A) || !al16(p.B)) return false;
  if (p.batch > 1 && (p.batch_a % 8 || p.batch_b % 8)) return false;
  return true;
}

static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (p.workspace) return hipErrorNotSupported;
  if (mfma_narrow_f16_can_run(p, 0)) return launch_mfma_narrow_f16(p, s);
  if ((p.sa_m != 1 && p.sa_k != 1) || (p.sb_n != 1 && p.sb_k != 1)) return hipErrorNotSupported;
  // (an operand with both strides 1 is a single row or column: either form reads it correctly)
  const bool a_kc = p.sa_k == 1, b_kc = p.sb_k == 1;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  const dim3 grid((unsigned)tiles, 1, p.batch), block(THREADS);
  const bool fast = exact(p, a_kc, b_kc);
#define CUASR_F16_LAUNCH(AK, BK_, G) launch_kernel((mfma_f16_kernel<AK, BK_, G>), grid, block, 0, s, p)
  if (fast) {
    if (a_kc) { if (b_kc) CUASR_F16_LAUNCH(true, true, false); else CUASR_F16_LAUNCH(true, false, false); }
    else { if (b_kc) CUASR_F16_LAUNCH(false, true, false); else CUASR_F16_LAUNCH(false, false, false); }
  } else {
    if (a_kc) { if (b_kc) CUASR_F16_LAUNCH(true, true, true); else CUASR_F16_LAUNCH(true, false, true); }
    else { if (b_kc) CUASR_F16_LAUNCH(false, true, true); else CUASR_F16_LAUNCH(false, false, true); }
  }
#undef CUASR_F16_LAUNCH
  return take_launch_status();
}

}  // namespace mfma_f16

launch_fn find_mfma_f16(int add_op, int mult_op) {
  return (add_op == kPlus && mult_op == kMultiplies) ? mfma_f16::launch : nullptr;
}

}  // namespace cuasr_amd
