// Plus-times on int8 operands with int32 accumulation, on the matrix cores.
//
// The reference carries threadblock cores for int8 operands built around the 4-way byte dot product
// (include/cuasr/gemm/threadblock/default_srmma_core_simt.h:733-1381: ElementA = ElementB = int8_t,
// InstructionShape 1 x 1 x 4), but never instantiates them.  On gfx950 the instruction for that job is
// v_mfma_i32_32x32x32_i8: a wave multiplies a 32 x 32 (rows x k) block of A by a 32 x 32 block of B, every lane
// supplying 16 consecutive k of one row (column).  Integer sums wrap modulo 2^32 whatever their order, so the
// result is bit-identical to the k-ascending reference loop.
//
// Tile: 256 threads (2 x 2 waves), 128 x 128 x 128; a wave holds 2 x 2 blocks of 32 x 32 (64 accumulator
// registers), two workgroups per compute unit.  The instruction is so fast (32 cycles for 65536 operations) that a
// k-tile is over in a thousand cycles, less than a trip to memory: the loads of tile t + 2 are issued before tile t
// is worked on and stay in registers for two tiles (two register sets, the tile loop unrolled by two), while LDS
// holds tiles t and t + 1.  LDS holds both panels k-contiguous, [x][128 k + 16 bytes of padding] (the padding makes
// the 16-byte fragment reads of 32 consecutive rows conflict-free).  Operands are staged through registers, which
// is where an operand whose rows (columns) are contiguous in memory gets transposed: a thread loads 16 x at 4
// consecutive k (four 16-byte loads), turns them with byte permutes into 16 words of 4 k each and writes those.
// Measured and not kept: a 256 x 256 tile (4 x 4 blocks per wave, 256 accumulator registers, one wave per SIMD),
// which halves the LDS reads per instruction: 0.75 against 1.02 POP/s at 4096^3 -- one wave per SIMD of compiled
// code has nothing to hide its own waits behind.
#include "semiring.h"

namespace cuasr_amd {

// the hand-scheduled form for whole 256 x 256 tiles of k-contiguous operands (mfma_direct_narrow.hip)
bool mfma_narrow_i8_can_run(const Problem &p, int units);
hipError_t launch_mfma_narrow_i8(const Problem &p, hipStream_t s);

namespace mfma_i8 {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 128, THREADS = 256, PITCH = BK + 16;
constexpr int KCH = BK / 16;  // 16-byte chunks along k

struct Smem {
  int8_t a[2][BM][PITCH];
  int8_t b[2][BN][PITCH];
};

// One operand's share of a k-tile (X x, BK k) on its way from memory to LDS.
//   KC (k contiguous in memory): chunks of 16 k of one x, written as they are.
//   otherwise (x contiguous):    units of 16 x by 4 k; four 16-byte loads, transposed in registers.
// GUARD: bytes beyond the extents read as zero (a zero factor adds nothing to a sum of products).
template <int X, bool KC, bool GUARD> struct Stager {
  static constexpr int CHUNKS = KCH * X / THREADS;                 // KC: 16-byte chunks per thread
  static constexpr int NUNITS = (X / 16) * (BK / 4);                // otherwise: units in the tile ...
  static constexpr int UNITS = (NUNITS + THREADS - 1) / THREADS;    // ... and per thread
  v4i r[KC ? CHUNKS : 4 * UNITS];
  // unit u -> (x, k) of its first element.  XB neighbouring lanes take neighbouring blocks of 16 x at one group of 4 k,
  // the next lanes the next groups of k: the lanes of one LDS store then write XB rows (16 apart: the same bank) at
  // 64 / XB consecutive words each -- a two-way bank conflict where x-fastest lanes had an eight-way one.
#ifndef CUASR_I8_XB
#define CUASR_I8_XB 2
#endif
  static constexpr int XB = CUASR_I8_XB;
  static_assert((X / 16) % XB == 0, "blocks of x split evenly");
  static __device__ __forceinline__ void where(int u, int &x, int &k) {
    const int lo = u % XB, kg = (u / XB) % (BK / 4), hi = u / (XB * (BK / 4));
    x = (hi * XB + lo) * 16;
    k = kg * 4;
  }

  static __device__ __forceinline__ v4i fetch(const int8_t *src, int first, int limit, bool live) {
    // 16 consecutive bytes; byte e is element first + e of a run that ends at `limit`
    if constexpr (!GUARD) {
      return *reinterpret_cast<const v4i *>(src);
    } else {
      v4i v = {0, 0, 0, 0};
      typedef int loose4 __attribute__((ext_vector_type(4), aligned(1)));  // (a vector load may start at any byte)
      if (live && first + 16 <= limit) {
        v = *reinterpret_cast<const loose4 *>(src);
      } else if (live) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int byte = (first + e < limit) ? (int)(unsigned char)src[e] : 0;
          v[e / 4] |= byte << (8 * (e % 4));
        }
      }
      return v;
    }
  }

  __device__ __forceinline__ void load(const int8_t *base, long long sx, long long sk, int x0, int k0, int xn, int kn) {
    if constexpr (KC) {
#pragma unroll
      for (int q = 0; q < CHUNKS; ++q) {
        const int c = threadIdx.x + q * THREADS, k = (c % KCH) * 16, x = c / KCH;
        r[q] = fetch(base + (long long)(x0 + x) * sx + (k0 + k), k0 + k, kn, x0 + x < xn);
      }
    } else {
#pragma unroll
      for (int q = 0; q < UNITS; ++q) {
        const int u = threadIdx.x + q * THREADS;
        if (u < NUNITS) {
          int x, k;
          where(u, x, k);
#pragma unroll
          for (int kk = 0; kk < 4; ++kk)
            r[4 * q + kk] = fetch(base + (x0 + x) + (long long)(k0 + k + kk) * sk, x0 + x, xn, k0 + k + kk < kn);
        }
      }
    }
  }

  __device__ __forceinline__ void store(int8_t (*panel)[PITCH]) const {
    if constexpr (KC) {
#pragma unroll
      for (int q = 0; q < CHUNKS; ++q) {
        const int c = threadIdx.x + q * THREADS, k = (c % KCH) * 16, x = c / KCH;
        *reinterpret_cast<v4i *>(&panel[x][k]) = r[q];
      }
    } else {
#pragma unroll
      for (int q = 0; q < UNITS; ++q) {
        const int u = threadIdx.x + q * THREADS;
        if (u < NUNITS) {
          int x, k;
          where(u, x, k);
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            // words d of the four loads hold x = 4d .. 4d+3 at k, k+1, k+2, k+3: a 4 x 4 byte transpose
            const unsigned a = r[4 * q + 0][d], b = r[4 * q + 1][d], c = r[4 * q + 2][d], e = r[4 * q + 3][d];
            const unsigned ab_lo = __builtin_amdgcn_perm(b, a, 0x05010400), ab_hi = __builtin_amdgcn_perm(b, a, 0x07030602);
            const unsigned ce_lo = __builtin_amdgcn_perm(e, c, 0x05010400), ce_hi = __builtin_amdgcn_perm(e, c, 0x07030602);
            *reinterpret_cast<unsigned *>(&panel[x + 4 * d + 0][k]) = __builtin_amdgcn_perm(ce_lo, ab_lo, 0x05040100);
            *reinterpret_cast<unsigned *>(&panel[x + 4 * d + 1][k]) = __builtin_amdgcn_perm(ce_lo, ab_lo, 0x07060302);
            *reinterpret_cast<unsigned *>(&panel[x + 4 * d + 2][k]) = __builtin_amdgcn_perm(ce_hi, ab_hi, 0x05040100);
            *reinterpret_cast<unsigned *>(&panel[x + 4 * d + 3][k]) = __builtin_amdgcn_perm(ce_hi, ab_hi, 0x07060302);
          }
        }
      }
    }
  }
};

template <bool A_KC, bool B_KC, bool GUARD>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void mfma_i8_kernel(Problem p) {
  __shared__ __attribute__((aligned(16))) Smem sm;
  select_batch<int32_t, int8_t>(p);
  const int tiles_n = (p.n + BN - 1) / BN;
  const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, half = lane >> 5;
  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const int8_t *A = reinterpret_cast<const int8_t *>(p.A), *B = reinterpret_cast<const int8_t *>(p.B);

  v16i acc[2][2];
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[bi][bj][e] = 0;

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
    for (int ks = 0; ks < BK / 32; ++ks) {
      v4i a[2], b[2];
#pragma unroll
      for (int bi = 0; bi < 2; ++bi) a[bi] = *reinterpret_cast<const v4i *>(&sm.a[s][wm * 64 + bi * 32 + l32][ks * 32 + half * 16]);
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) b[bj] = *reinterpret_cast<const v4i *>(&sm.b[s][wn * 64 + bj * 32 + l32][ks * 32 + half * 16]);
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) acc[bi][bj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[bi], b[bj], acc[bi][bj], 0, 0, 0);
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
  const EpilogueScalars<int32_t> sc = resolve_scalars<int32_t>(p, kMultiplies);
  int32_t *ws = p.workspace ? reinterpret_cast<int32_t *>(p.workspace) + (long long)blockIdx.y * p.m * p.n : nullptr;
  const int32_t *C = reinterpret_cast<const int32_t *>(p.C);
  int32_t *D = reinterpret_cast<int32_t *>(p.D);
  // A store instruction writes 128 consecutive bytes of two rows; the two blocks of a block row are stored register by
  // register, so that consecutive instructions write consecutive pieces of the same rows, and a block row's source
  // elements are requested together, before any of its results is stored (D may be C, so the compiler cannot move a
  // load of C above a store to D by itself)
#pragma unroll
  for (int bi = 0; bi < 2; ++bi) {
    auto row_of = [&](int e) { return m0 + wm * 64 + bi * 32 + 8 * (e / 4) + 4 * half + (e % 4); };
    auto inside = [&](int row, int col) { return !GUARD || ((unsigned)row < (unsigned)p.m && (unsigned)col < (unsigned)p.n); };
    int32_t src[16][2];
    if (!ws && sc.source_needed) {
#pragma unroll
      for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj) {
          const int row = row_of(e), col = n0 + wn * 64 + bj * 32 + l32;
          src[e][bj] = inside(row, col) ? C[(long long)row * p.ldc + col] : 0;
        }
    }
#pragma unroll
    for (int e = 0; e < 16; ++e)
#pragma unroll
      for (int bj = 0; bj < 2; ++bj) {
        const int row = row_of(e), col = n0 + wn * 64 + bj * 32 + l32;
        if (!inside(row, col)) continue;
        const int32_t v = acc[bi][bj][e];
        if (ws) {
          ws[(long long)row * p.n + col] = v;
        } else {
          // unsigned arithmetic: the same bits as the two's-complement result, with no overflow to reason about
          uint32_t out = (uint32_t)sc.alpha * (uint32_t)v;
          if (sc.source_needed) out += (uint32_t)sc.beta * (uint32_t)src[e][bj];
          D[(long long)row * p.ldd + col] = (int32_t)out;
        }
      }
  }
}

// whole tiles of 16-byte aligned operands: the unguarded kernel
static bool exact(const Problem &p, bool a_kc, bool b_kc) {
  auto al16 = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  if (p.m % BM || p.n % BN || p.k % BK || p.k == 0) return false;
  if (p.workspace && p.k_per_slice % BK) return false;
  if ((a_kc ? p.sa_m : p.sa_k) % 16 || (b_kc ? p.sb_n : p.sb_k) % 16) return false;
  if (!al16(p.A) || !al16(p.B)) return false;
  if (p.batch > 1 && (p.batch_a % 16 || p.batch_b % 16)) return false;
  return true;
}

static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (mfma_narrow_i8_can_run(p, 0)) return launch_mfma_narrow_i8(p, s);
  if ((p.sa_m != 1 && p.sa_k != 1) || (p.sb_n != 1 && p.sb_k != 1)) return hipErrorNotSupported;
  // (an operand with both strides 1 is a single row or column: either form reads it correctly)
  const bool a_kc = p.sa_k == 1, b_kc = p.sb_k == 1;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + BN - 1) / BN);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  const dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1, p.batch), block(THREADS);
  const bool fast = exact(p, a_kc, b_kc);
#define CUASR_I8_LAUNCH(AK, BK_, G) launch_kernel((mfma_i8_kernel<AK, BK_, G>), grid, block, 0, s, p)
  if (fast) {
    if (a_kc) { if (b_kc) CUASR_I8_LAUNCH(true, true, false); else CUASR_I8_LAUNCH(true, false, false); }
    else { if (b_kc) CUASR_I8_LAUNCH(false, true, false); else CUASR_I8_LAUNCH(false, false, false); }
  } else {
    if (a_kc) { if (b_kc) CUASR_I8_LAUNCH(true, true, true); else CUASR_I8_LAUNCH(true, false, true); }
    else { if (b_kc) CUASR_I8_LAUNCH(false, true, true); else CUASR_I8_LAUNCH(false, false, true); }
  }
#undef CUASR_I8_LAUNCH
  return take_launch_status();
}

}  // namespace mfma_i8

launch_fn find_mfma_i8(int add_op, int mult_op) {
  return (add_op == kPlus && mult_op == kMultiplies) ? mfma_i8::launch : nullptr;
}

}  // namespace cuasr_amd
