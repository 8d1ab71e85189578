// Vector-ALU tile for element type binary16 (half precision), two output columns per register: the kernel and
// its launcher, instantiated by valu_f16.hip (binary16 operands) and valu_i8.hip (int8 operands; or-and on
// float / double operands).
//
// The reference names half precision as an aim only (README.md:11); its templates, instantiated
// with a half type for every element, would round each operator's result to binary16
// (arch/srmma.h:65-92: d = add(c, mult(a, b)) in ElementC).  So does this tile: every term is one
// packed add (or max, min, mul) and every fold one packed min / max / add on two binary16 values.
//
// What gfx950 gives for it (cuasr_amd/issue_probe.py, "mix_f16"): a packed binary16 instruction
// issues every 4.2 cycles per SIMD, twice as long as a 4-byte one, so two terms per instruction buy
// no rate by themselves (99.6 against 97 TOPS for the bare loops) -- but LDS reads, waits and address
// arithmetic issue beneath the 4-cycle instructions for free, two waves per SIMD already reach that
// rate, and the operands are half as many bytes.  Hence a plain compiled loop, staged through
// registers, which can also transpose on the way to LDS: one kernel serves every layout.
//
// Tile: 256 threads, 128 rows x 256 columns x 32 k.  A thread holds 8 rows x 16 columns (two groups
// of 8 consecutive columns, 128 apart) as 64 registers of two columns each.  LDS: A panel [k][128],
// B panel [k][256], both with the output direction contiguous, two stages.  Per k a thread reads one
// 16-byte vector of A (its 8 rows; the instruction's half-word selects broadcast one of them) and two
// of B, and issues 64 packed adds + 32 three-input packed minima for 128 terms.
// Outputs too small to give the 256 compute units two such tiles each take smaller ones of the same kernel, guarded
// form only: 64 x 128 (4 rows and one column group per thread); below that 32 x 128 and 16 x 128 with every k-tile
// shared out between the four waves (min, max, or), or 32 x 128 with 2 rows per thread (plus, whose order counts).
//
// int8 operands (CUASR_AMD_I8: int8 A and B, int32 everything else) ride on the same kernel for min-plus,
// max-plus, min-max and max-min: every int8 value, and every sum of two, is a binary16 value, so the terms and
// their minima are exact; the operands are converted on their way to LDS, the accumulators on their way out,
// and the epilogue (the caller's additive identity included) is integer arithmetic.  On the vector ALU that is
// twice the rate integers get (three-input integer minima and byte-selecting adds issue at half rate).
// min-times, max-times and the bitwise pairs on int8 operands use the kernel with int16 lanes (int16_lanes below).
#pragma once
#include "semiring.h"

namespace cuasr_amd {
namespace half_tile {

typedef half_t h2 __attribute__((ext_vector_type(2)));
typedef half_t h8 __attribute__((ext_vector_type(8)));

constexpr int BK = 32, THREADS = 256;

template <int BM, int BN> struct Smem {
  half_t a[2][BK][BM];
  half_t b[2][BK][BN];
};

template <int OP> __device__ __forceinline__ h2 pk(h2 l, h2 r) {
  if constexpr (OP == kPlus) return l + r;
  else if constexpr (OP == kMultiplies) return l * r;
  else if constexpr (OP == kMinimum) return __builtin_elementwise_min(l, r);
  else return __builtin_elementwise_max(l, r);
}

// acc <- add(acc, mult(a0, b0), mult(a1, b1)), the two terms in this order
// or-and: `lhs && rhs`, `lhs || rhs` (functional.h:212, :252) only look at whether an operand is zero, so the
// panels go to LDS as 16-bit masks (all ones / zero) and a term is one three-input bit operation acc | (a & b)
// on a register of two masks
template <int ADD, int MUL> struct masked : std::integral_constant<bool, ADD == kLogicalOr && MUL == kLogicalAnd> {};
__device__ __forceinline__ h2 or_and_pair(h2 acc, h2 a, h2 b) {
  return __builtin_bit_cast(h2, or_and_term(__builtin_bit_cast(uint32_t, acc), __builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b)));
}

// int8 operands under min-times / max-times: a product of two int8 values is a 16-bit integer (|a b| <= 16384) but no
// binary16 value, so the lanes hold int16 and the instructions are the packed 16-bit integer ones (v_pk_mul_lo_u16,
// v_pk_min_i16 / v_pk_max_i16; there is no three-input packed integer minimum: four instructions per four terms).
// The bitwise pairs on int8 operands (xor-and, or-and on bits) use the same lanes: the operators act on the widened
// values, and the bitwise and / xor / or of sign-extended 8-bit values are the sign extensions of the 8-bit results,
// at 16 bits as at 32; a term is one three-input bit operation on a register of two lanes.
typedef short s2 __attribute__((ext_vector_type(2)));
template <int ADD, int MUL, typename TI> struct int16_lanes
    : std::integral_constant<bool, std::is_same<TI, int8_t>::value &&
                                       ((MUL == kMultiplies && (ADD == kMinimum || ADD == kMaximum)) ||
                                        (MUL == kBitAnd && (ADD == kBitXor || ADD == kBitOr)))> {};
template <int ADD> __device__ __forceinline__ h2 int16_fold(h2 l, h2 r) {
  const s2 x = __builtin_bit_cast(s2, l), y = __builtin_bit_cast(s2, r);
  if constexpr (ADD == kBitXor) return __builtin_bit_cast(h2, x ^ y);
  else if constexpr (ADD == kBitOr) return __builtin_bit_cast(h2, x | y);
  else return __builtin_bit_cast(h2, ADD == kMinimum ? __builtin_elementwise_min(x, y) : __builtin_elementwise_max(x, y));
}
__device__ __forceinline__ h2 int16_product(h2 a, h2 b) { return __builtin_bit_cast(h2, __builtin_bit_cast(s2, a) * __builtin_bit_cast(s2, b)); }
template <int ADD, int MUL> __device__ __forceinline__ h2 int16_term(h2 acc, h2 a, h2 b) {
  if constexpr (MUL == kBitAnd) {
    const uint32_t x = __builtin_bit_cast(uint32_t, acc), u = __builtin_bit_cast(uint32_t, a), v = __builtin_bit_cast(uint32_t, b);
    return __builtin_bit_cast(h2, ADD == kBitXor ? xor_and_term(x, u, v) : or_and_term(x, u, v));
  } else {
    return int16_fold<ADD>(acc, int16_product(a, b));
  }
}

template <int ADD, int MUL, bool I16 = false> __device__ __forceinline__ void two_terms(h2 &acc, h2 a0, h2 b0, h2 a1, h2 b1) {
  if constexpr (I16) {
    acc = int16_term<ADD, MUL>(int16_term<ADD, MUL>(acc, a0, b0), a1, b1);
    return;
  }
  if constexpr (masked<ADD, MUL>::value) {
    acc = or_and_pair(or_and_pair(acc, a0, b0), a1, b1);
    return;
  }
  const h2 t0 = pk<MUL>(a0, b0), t1 = pk<MUL>(a1, b1);
  // the three-input forms (v_pk_minimum3_f16 / v_pk_maximum3_f16) differ from min / max only on NaN
  if constexpr (ADD == kMinimum) acc = __builtin_elementwise_minimum(__builtin_elementwise_minimum(acc, t0), t1);
  else if constexpr (ADD == kMaximum) acc = __builtin_elementwise_maximum(__builtin_elementwise_maximum(acc, t0), t1);
  else acc = pk<ADD>(pk<ADD>(acc, t0), t1);
}
template <int ADD, int MUL, bool I16 = false> __device__ __forceinline__ void one_term(h2 &acc, h2 a, h2 b) {
  if constexpr (I16) acc = int16_term<ADD, MUL>(acc, a, b);
  else if constexpr (masked<ADD, MUL>::value) acc = or_and_pair(acc, a, b);
  else acc = pk<ADD>(acc, pk<MUL>(a, b));
}

// add(l, r) of two partial accumulators (or-and: of two masks)
template <int ADD, int MUL, bool I16 = false> __device__ __forceinline__ h2 fold(h2 l, h2 r) {
  if constexpr (I16) return int16_fold<ADD>(l, r);
  else if constexpr (masked<ADD, MUL>::value) return __builtin_bit_cast(h2, __builtin_bit_cast(uint32_t, l) | __builtin_bit_cast(uint32_t, r));
  else return pk<ADD>(l, r);
}

__device__ __forceinline__ h2 both(half_t v) { return h2{v, v}; }
__device__ __forceinline__ h2 pair_of(const h8 &v, int j) { return h2{v[2 * j], v[2 * j + 1]}; }
template <int N> struct frag_of { typedef half_t type __attribute__((ext_vector_type(N))); };
// what C, D, the scalars and the workspace hold for operands of type TI; 8 of them, 8 operands
template <typename TI> struct out_of { typedef half_t type; };
template <> struct out_of<int8_t> { typedef int32_t type; };
template <> struct out_of<float> { typedef float type; };    // (or-and only: the operands go to LDS as masks)
template <> struct out_of<double> { typedef double type; };
template <> struct out_of<int32_t> { typedef int32_t type; };
template <> struct out_of<uint32_t> { typedef uint32_t type; };
template <typename T> struct vec8 { typedef T type __attribute__((ext_vector_type(8), aligned(sizeof(T) * 8 < 16 ? sizeof(T) * 8 : 16))); };
template <typename TI> __device__ __forceinline__ half_t to_half(TI v) { return half_t(float(v)); }
template <> __device__ __forceinline__ half_t to_half<half_t>(half_t v) { return v; }

// One operand's share of a k-tile on its way from memory to LDS.  The panel is X wide (X = BM for A, BN
// for B); a chunk is 8 elements: of one k and 8 consecutive x when x is the contiguous direction in
// memory, of one x and 8 consecutive k otherwise (KC).  CHUNKS chunks per thread.
template <int X, bool KC, bool GUARD, typename TI, bool MASK = false, bool I16 = false> struct Stager {
  // what goes to LDS for one operand: its binary16 value, or (MASK) all ones / zero for non-zero / zero, or (I16)
  // the 16-bit integer
  static __device__ __forceinline__ half_t staged(TI v) {
    if constexpr (I16) return __builtin_bit_cast(half_t, (short)v);
    else if constexpr (MASK) return __builtin_bit_cast(half_t, (unsigned short)(truth(v) ? 0xffff : 0));
    else return to_half<TI>(v);
  }
  typedef typename vec8<TI>::type raw8;
  // the same eight operands at any element boundary (the hardware takes a vector load at any address)
  typedef TI loose8 __attribute__((ext_vector_type(8), aligned(sizeof(TI))));
  static constexpr int TOTAL = X * BK / 8, CHUNKS = (TOTAL + THREADS - 1) / THREADS;  // (a small panel leaves threads idle)
  h8 r[CHUNKS];

  // chunk c -> (x, k) of its first element, tile-relative
  static __device__ __forceinline__ void where(int c, int &x, int &k) {
    if constexpr (KC) {
      // KL neighbouring lanes take neighbouring chunks of k of one x, the next lanes the next x: the 2-byte stores of
      // one instruction then go to KL rows of the panel (8 apart: the same banks) at 64 / KL consecutive x each
#ifndef CUASR_HALF_KL
#define CUASR_HALF_KL 2
#endif
      constexpr int KL = CUASR_HALF_KL;
      static_assert((BK / 8) % KL == 0, "chunks of k split evenly");
      k = ((c / (KL * X)) * KL + c % KL) * 8;
      x = (c / KL) % X;
    } else {
      x = (c % (X / 8)) * 8;
      k = c / (X / 8);
    }
  }

  // base: the operand's element (x = 0, k = 0); sx, sk: element strides; x0, k0: the tile's origin;
  // xn, kn: the extents (elements beyond them read as zero and are never used in a result that is stored).
  // In the guarded form a chunk that lies wholly inside the extents is read as a vector all the same, at whatever
  // element boundary it starts; only chunks across an edge are read element by element
  template <typename V> static __device__ __forceinline__ h8 widen(const V v) {
    h8 h;
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = staged(v[e]);
    return h;
  }
  __device__ __forceinline__ void load(const TI *base, long long sx, long long sk, int x0, int k0, int xn, int kn) {
#pragma unroll
    for (int q = 0; q < CHUNKS; ++q) {
      if (TOTAL % THREADS && (int)threadIdx.x + q * THREADS >= TOTAL) break;
      int x, k;
      where(threadIdx.x + q * THREADS, x, k);
      const TI *src = base + (long long)(x0 + x) * sx + (long long)(k0 + k) * sk;
      if constexpr (!GUARD) {
        r[q] = widen(*reinterpret_cast<const raw8 *>(src));
      } else {
        const bool whole = KC ? (x0 + x < xn && k0 + k + 8 <= kn) : (x0 + x + 8 <= xn && k0 + k < kn);
        if (whole) {
          r[q] = widen(*reinterpret_cast<const loose8 *>(src));
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int xe = x0 + x + (KC ? 0 : e), ke = k0 + k + (KC ? e : 0);
            r[q][e] = (xe < xn && ke < kn) ? staged(src[(KC ? sk : sx) * e]) : half_t(0);
          }
        }
      }
    }
  }

  __device__ __forceinline__ void store(half_t (*panel)[X]) const {
#pragma unroll
    for (int q = 0; q < CHUNKS; ++q) {
      if (TOTAL % THREADS && (int)threadIdx.x + q * THREADS >= TOTAL) break;
      int x, k;
      where(threadIdx.x + q * THREADS, x, k);
      if constexpr (KC) {
#pragma unroll
        for (int e = 0; e < 8; ++e) panel[k + e][x] = r[q][e];
      } else {
        *reinterpret_cast<h8 *>(&panel[k][x]) = r[q];
      }
    }
  }
};

// the last product of a k range that is zero (acc itself when there is none); not inlined: it runs after the main loop
static __device__ __attribute__((noinline)) half_t last_zero_product(const half_t *a_row, long long sa_k, const half_t *b_col,
                                                                     long long sb_k, int kcount, half_t acc) {
  // sixteen k at a time, so that the loads of a step are in flight together (one lane scans alone: a step costs a
  // memory latency whatever it fetches)
  int kk = kcount - 1;
  for (; kk >= 15; kk -= 16) {
    half_t prod[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) prod[u] = a_row[(long long)(kk - u) * sa_k] * b_col[(long long)(kk - u) * sb_k];
#pragma unroll
    for (int u = 0; u < 16; ++u)
      if (prod[u] == half_t(0)) return prod[u];
  }
  for (; kk >= 0; --kk) {
    const half_t prod = a_row[(long long)kk * sa_k] * b_col[(long long)kk * sb_k];
    if (prod == half_t(0)) return prod;
  }
  return acc;
}

// TR rows and NG groups of 8 columns per thread.  KS = 1: the 256 threads are 16 x 16, the tile 16 TR x 128 NG.
// KS = 4 (adds that do not care about order, and about repetition of the value every part starts from -- min, max,
// or, and xor, which starts from zero): a wave is 16 x 4 threads and covers a
// tile of 4 TR x 128 NG by itself, each of the four waves takes a quarter of every k-tile, and the four partial
// accumulators meet in LDS before the epilogue.  A small output then still gives every SIMD a wave, and the wave
// the full tile's work per LDS read.
template <int ADD, int MUL, bool A_KC, bool B_KC, bool GUARD, int TR = 8, int NG = 2, typename TI = half_t, int KS = 1, int AHEAD = 1>
__global__ __launch_bounds__(THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void half_tile_kernel(Problem p) {
  static_assert(KS == 1 || (KS == 4 && ADD != kPlus && TR % KS == 0), "k is shared out between waves only for order-free adds");
  constexpr int TY = 16 / KS, BM = TY * TR, BN = 128 * NG;
  constexpr int KW = BK / KS;        // k per tile and part
  constexpr int IR = TR / KS;        // rows of its accumulators that a thread takes through the epilogue
  constexpr bool BYTES = std::is_same<TI, int8_t>::value;
  constexpr bool ZERO_SIGN = !BYTES && MUL == kMultiplies && (ADD == kMinimum || ADD == kMaximum);
  constexpr bool MASKED = masked<ADD, MUL>::value;
  constexpr bool I16 = int16_lanes<ADD, MUL, TI>::value;
  typedef typename out_of<TI>::type TO;
  typedef typename vec8<TO>::type out8;
  typedef typename frag_of<TR>::type rows_t;
  typedef Smem<BM, BN> panels_t;
  typedef h2 partials_t[KS][TR * 4 * NG][THREADS / KS];   // [part][accumulator][lane]
  constexpr size_t lds_bytes = KS > 1 && sizeof(partials_t) > sizeof(panels_t) ? sizeof(partials_t) : sizeof(panels_t);
  __shared__ __attribute__((aligned(16))) unsigned char lds[lds_bytes];   // the panels, and after the last k-tile the partials
  panels_t &sm = *reinterpret_cast<panels_t *>(lds);
  select_batch<TO, TI>(p);
  const int tiles_n = (p.n + BN - 1) / BN;
  const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;
  const int tx = threadIdx.x % 16, ty = (threadIdx.x / 16) % TY;
  const int part = KS > 1 ? threadIdx.x / (THREADS / KS) : 0, kf = part * KW;
  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const TI *A = reinterpret_cast<const TI *>(p.A), *B = reinterpret_cast<const TI *>(p.B);
  // int8 operands: the loop starts from the binary16 infinity of its add; the caller's identity joins at the end
  // (or-and: the loop ors masks, starting from none; the caller's identity joins at the end as well)
  const half_t ident = MASKED ? half_t(0)
                       : I16   ? __builtin_bit_cast(half_t, (short)(ADD == kMinimum ? 32767 : ADD == kMaximum ? -32768 : 0))
                       : BYTES ? half_t(ADD == kMinimum ? __builtin_inff() : -__builtin_inff()) : scalar_as<half_t>(p.add_identity);

  h2 acc[TR][4 * NG];  // [row][column pair]: pairs 0..3 = columns tx*8 .. +7, pairs 4..7 = the same 128 further on
#pragma unroll
  for (int i = 0; i < TR; ++i)
#pragma unroll
    for (int j = 0; j < 4 * NG; ++j) acc[i][j] = both(ident);

  // AHEAD = 2: the loads of k-tile t + 2 are issued before the terms of tile t, into the registers that tile t
  // passed through (a workgroup alone on its compute unit has nobody to hide a memory latency behind)
  Stager<BM, A_KC, GUARD, TI, MASKED, I16> sa[AHEAD];
  Stager<BN, B_KC, GUARD, TI, MASKED, I16> sb[AHEAD];
  const int tiles_k = ke > kb ? (ke - kb + BK - 1) / BK : 0;
  auto fetch = [&](auto set, int t) {
    sa[set.value].load(A, p.sa_m, p.sa_k, m0, kb + t * BK, p.m, ke);
    sb[set.value].load(B, p.sb_n, p.sb_k, n0, kb + t * BK, p.n, ke);
  };
  if (tiles_k > 0) {
    fetch(std::integral_constant<int, 0>(), 0);
    sa[0].store(sm.a[0]);
    sb[0].store(sm.b[0]);
    if (AHEAD == 2 && tiles_k > 1) fetch(std::integral_constant<int, AHEAD - 1>(), 1);
  }
  __syncthreads();
  // k-tile t, whose operands passed through register set `set`; tile t + 1 sits in the other one (AHEAD = 2)
  auto tile = [&](auto set, int t) {
    constexpr int next = (set.value + 1) % AHEAD;
    const int s = t & 1, k0 = kb + t * BK;
    if (t + AHEAD < tiles_k) fetch(set, t + AHEAD);
    const half_t(*pa)[BM] = sm.a[s];
    const half_t(*pb)[BN] = sm.b[s];
    if (!GUARD || ke - k0 >= BK) {
#pragma unroll 2
      for (int kk = kf; kk < kf + KW; kk += 2) {
        const rows_t a0 = *reinterpret_cast<const rows_t *>(&pa[kk][ty * TR]), a1 = *reinterpret_cast<const rows_t *>(&pa[kk + 1][ty * TR]);
        h8 b0[NG], b1[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          b0[g] = *reinterpret_cast<const h8 *>(&pb[kk][g * 128 + tx * 8]);
          b1[g] = *reinterpret_cast<const h8 *>(&pb[kk + 1][g * 128 + tx * 8]);
        }
#pragma unroll
        for (int i = 0; i < TR; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < NG; ++g)
              two_terms<ADD, MUL, I16>(acc[i][4 * g + j], both(a0[i]), pair_of(b0[g], j), both(a1[i]), pair_of(b1[g], j));
      }
    } else {
      for (int kk = kf; kk < min(kf + KW, ke - k0); ++kk) {  // the ragged last k-tile
        const rows_t a0 = *reinterpret_cast<const rows_t *>(&pa[kk][ty * TR]);
        h8 b0[NG];
#pragma unroll
        for (int g = 0; g < NG; ++g) b0[g] = *reinterpret_cast<const h8 *>(&pb[kk][g * 128 + tx * 8]);
#pragma unroll
        for (int i = 0; i < TR; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int g = 0; g < NG; ++g) one_term<ADD, MUL, I16>(acc[i][4 * g + j], both(a0[i]), pair_of(b0[g], j));
      }
    }
    if (t + 1 < tiles_k) {
      sa[next].store(sm.a[s ^ 1]);
      sb[next].store(sm.b[s ^ 1]);
    }
    __syncthreads();
  };
  for (int t = 0; t < tiles_k; t += AHEAD) {
    tile(std::integral_constant<int, 0>(), t);
    if (AHEAD == 2 && t + 1 < tiles_k) tile(std::integral_constant<int, AHEAD - 1>(), t + 1);
  }

  // ---- the parts' accumulators meet: part q finishes rows q IR .. q IR + IR - 1 of every thread's TR
  h2 fin[IR][4 * NG];
  if constexpr (KS == 1) {
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
      for (int j = 0; j < 4 * NG; ++j) fin[i][j] = acc[i][j];
  } else {
    partials_t &red = *reinterpret_cast<partials_t *>(lds);   // (every wave is past the last k-tile's barrier)
    const int lane = threadIdx.x % (THREADS / KS);
#pragma unroll
    for (int i = 0; i < TR; ++i)
#pragma unroll
      for (int j = 0; j < 4 * NG; ++j) red[part][i * 4 * NG + j][lane] = acc[i][j];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < IR; ++i)
#pragma unroll
      for (int j = 0; j < 4 * NG; ++j) {
        h2 v = red[0][(part * IR + i) * 4 * NG + j][lane];
#pragma unroll
        for (int w = 1; w < KS; ++w) v = fold<ADD, MUL, I16>(v, red[w][(part * IR + i) * 4 * NG + j][lane]);
        fin[i][j] = v;
      }
  }

  // ---- epilogue: D = add(mult(alpha, acc), mult(beta, C)), or the raw accumulators of a k-slice
  const EpilogueScalars<TO> e = resolve_scalars<TO>(p, MUL);
  TO *ws = p.workspace ? reinterpret_cast<TO *>(p.workspace) + (long long)blockIdx.y * p.m * p.n : nullptr;
  const TO *C = reinterpret_cast<const TO *>(p.C);
  TO *D = reinterpret_cast<TO *>(p.D);
#pragma unroll
  for (int i = 0; i < IR; ++i) {
    const int row = m0 + ty * TR + part * IR + i;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const int col = n0 + g * 128 + tx * 8;
      out8 v;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const half_t a = fin[i][g * 4 + j / 2][j % 2];
        if constexpr (MASKED) {
          // the reference's accumulator after k > 0 terms: 1 if any term or the identity is non-zero, else 0
          const bool any = __builtin_bit_cast(unsigned short, a) != 0 || truth(e.ident);
          v[j] = tiles_k > 0 ? TO(any ? 1 : 0) : e.ident;
        } else if constexpr (I16) v[j] = tiles_k > 0 ? Op<ADD>::apply(e.ident, TO(__builtin_bit_cast(short, a))) : e.ident;
        else if constexpr (BYTES) v[j] = tiles_k > 0 ? Op<ADD>::apply(e.ident, TO(float(a))) : e.ident;  // (an exact integer)
        else v[j] = a;
        if constexpr (ZERO_SIGN) {
          // a minimum / maximum that is zero: the reference's comparison keeps the newer of two equal operands
          // (host_srgemm.h:87 with functional.h:132, :172), so its zero has the sign of the LAST zero product of
          // the k range, where the packed instruction keeps -0.  Looked up for the few accumulators that end at zero.
          if (a == half_t(0) && (unsigned)row < (unsigned)p.m && (unsigned)(col + j) < (unsigned)p.n)
            v[j] = last_zero_product(A + (long long)row * p.sa_m + (long long)kb * p.sa_k, p.sa_k,
                                     B + (long long)(col + j) * p.sb_n + (long long)kb * p.sb_k, p.sb_k, ke - kb, a);
        }
      }
      if (ws) {
        if constexpr (!GUARD) {
          *reinterpret_cast<out8 *>(ws + (long long)row * p.n + col) = v;
        } else {
#pragma unroll
          for (int x = 0; x < 8; ++x)
            if ((unsigned)row < (unsigned)p.m && (unsigned)(col + x) < (unsigned)p.n) ws[(long long)row * p.n + col + x] = v[x];
        }
        continue;
      }
      out8 c;
#pragma unroll
      for (int x = 0; x < 8; ++x) c[x] = e.ident;
      if (e.source_needed) {
        if constexpr (!GUARD) {
          c = *reinterpret_cast<const out8 *>(C + (long long)row * p.ldc + col);
        } else {
#pragma unroll
          for (int x = 0; x < 8; ++x)
            if ((unsigned)row < (unsigned)p.m && (unsigned)(col + x) < (unsigned)p.n) c[x] = C[(long long)row * p.ldc + col + x];
        }
      }
      out8 out;
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        out[x] = Op<MUL>::apply(e.alpha, v[x]);
        if (e.source_needed) out[x] = fold_epilogue<ADD, MUL>(out[x], Op<MUL>::apply(e.beta, c[x]));
      }
      if constexpr (!GUARD) {
        *reinterpret_cast<out8 *>(D + (long long)row * p.ldd + col) = out;
      } else {
#pragma unroll
        for (int x = 0; x < 8; ++x)
          if ((unsigned)row < (unsigned)p.m && (unsigned)(col + x) < (unsigned)p.n) D[(long long)row * p.ldd + col + x] = out[x];
      }
    }
  }
}

// whole tiles, whole vectors at vector boundaries everywhere: the unguarded kernel
template <typename TI> static bool exact(const Problem &p, bool a_kc, bool b_kc) {
  typedef typename out_of<TI>::type TO;
  constexpr uintptr_t in_bytes = 8 * sizeof(TI) < 16 ? 8 * sizeof(TI) : 16;   // a chunk of 8 operands: one or more vector loads
  constexpr long long out_step = 16 / sizeof(TO);           // elements of C / D per 16 bytes
  auto al = [](const void *q, uintptr_t to) { return reinterpret_cast<uintptr_t>(q) % to == 0; };
  if (p.m % 128 || p.n % 256 || p.k % BK || p.k == 0) return false;
  if (p.workspace && (p.k_per_slice % BK || !al(p.workspace, 16))) return false;
  if ((a_kc ? p.sa_m : p.sa_k) % 8 || (b_kc ? p.sb_n : p.sb_k) % 8) return false;
  if (!al(p.A, in_bytes) || !al(p.B, in_bytes) || !al(p.D, 16) || p.ldd % out_step) return false;
  if (p.C && (!al(p.C, 16) || p.ldc % out_step)) return false;
  if (p.batch > 1 && (p.batch_a % 8 || p.batch_b % 8 || p.batch_c % out_step || p.batch_d % out_step)) return false;
  return true;
}

template <int ADD, int MUL, bool GUARD, int TR, int NG, typename TI, int KS = 1, int AHEAD = 1>
static hipError_t launch_tile(const Problem &p, bool a_kc, bool b_kc, hipStream_t s) {
  constexpr int BM = 16 / KS * TR;
  const long long tiles = (long long)((p.m + BM - 1) / BM) * ((p.n + 128 * NG - 1) / (128 * NG));
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  const dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1, p.batch), block(THREADS);
#define CUASR_HALF_LAUNCH(AK, BK_) launch_kernel((half_tile_kernel<ADD, MUL, AK, BK_, GUARD, TR, NG, TI, KS, AHEAD>), grid, block, 0, s, p)
  if (a_kc) { if (b_kc) CUASR_HALF_LAUNCH(true, true); else CUASR_HALF_LAUNCH(true, false); }
  else { if (b_kc) CUASR_HALF_LAUNCH(false, true); else CUASR_HALF_LAUNCH(false, false); }
#undef CUASR_HALF_LAUNCH
  return take_launch_status();
}

template <int ADD, int MUL, typename TI = half_t> static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  // one direction of each operand is contiguous (the C ABI produces nothing else)
  if ((p.sa_m != 1 && p.sa_k != 1) || (p.sb_n != 1 && p.sb_k != 1)) return hipErrorNotSupported;
  const bool a_kc = p.sa_m != 1, b_kc = p.sb_n != 1;
  // Which tile.  A compute unit holds at most two of these workgroups (two waves per SIMD) and works two off
  // faster than one, but not twice as fast (a packed instruction occupies the vector ALU for four cycles: one
  // wave per SIMD keeps it busy most of the time); smaller tiles do less work per LDS read and per barrier.
  // `alone` / `paired`: the chip's rate in TOPS with one / two workgroups of that tile on every compute unit
  // (min-plus, measured from 512^3 to 4096^3).  The time is about that of the rounds of 512 workgroups at the
  // paired rate plus a last round at whichever rate its size gives; the tile with the smallest wins.
  auto cost = [&](int bm, int bn, long long alone, long long paired) {
    const long long groups = (long long)((p.m + bm - 1) / bm) * ((p.n + bn - 1) / bn) * (p.workspace ? p.slices : 1) * p.batch;
    const long long rest = groups % 512, area = (long long)bm * bn;
    return groups / 512 * (512 * area / paired) + (rest > 256 ? 512 * area / paired : rest > 0 ? 256 * area / alone : 0);
  };
  // (or-and: the full tile's term is half an instruction; the smaller tiles are bound by what surrounds the terms)
  const bool bits = masked<ADD, MUL>::value || MUL == kBitAnd;
  const long long full = bits ? cost(128, 256, 95, 128) : cost(128, 256, 63, 83), mid = bits ? cost(64, 128, 50, 76) : cost(64, 128, 50, 68);
  if constexpr (ADD == kPlus) {
    // the sum's order is the reference's: every k-tile whole in one thread
    const long long small = cost(32, 128, 36, 55);
    if (full <= mid && full <= small) {
      if (exact<TI>(p, a_kc, b_kc)) return launch_tile<ADD, MUL, false, 8, 2, TI>(p, a_kc, b_kc, s);
      return launch_tile<ADD, MUL, true, 8, 2, TI>(p, a_kc, b_kc, s);
    }
    if (mid <= small) return launch_tile<ADD, MUL, true, 4, 1, TI>(p, a_kc, b_kc, s);
    return launch_tile<ADD, MUL, true, 2, 1, TI>(p, a_kc, b_kc, s);
  } else {
    // min, max, or: the small tiles share every k-tile out between the four waves (1024^3 min-plus: 47 - 49 TOPS
    // against 33 - 37 with whole k-tiles per thread; 512^3: 13 - 14 against 8)
    const long long sliced = cost(32, 128, 43, 62), narrow = cost(16, 128, 35, 48);
    if (full <= mid && full <= sliced && full <= narrow) {
      if (exact<TI>(p, a_kc, b_kc)) return launch_tile<ADD, MUL, false, 8, 2, TI>(p, a_kc, b_kc, s);
      return launch_tile<ADD, MUL, true, 8, 2, TI>(p, a_kc, b_kc, s);
    }
    if (mid <= sliced && mid <= narrow) return launch_tile<ADD, MUL, true, 4, 1, TI>(p, a_kc, b_kc, s);
    if (sliced <= narrow) return launch_tile<ADD, MUL, true, 8, 1, TI, 4, 2>(p, a_kc, b_kc, s);
    return launch_tile<ADD, MUL, true, 4, 1, TI, 4, 2>(p, a_kc, b_kc, s);
  }
}

}  // namespace half_tile

}  // namespace cuasr_amd
