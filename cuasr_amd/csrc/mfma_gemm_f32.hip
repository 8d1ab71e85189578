// plus-times ("control") semiring for float on the matrix cores:
//     D = alpha * (A . B) + beta * C      with v_mfma_f32_32x32x2_f32
//
// The only semiring a matrix instruction computes as is.  Replaces, for this
// pair, the reference's SIMT kernel (include/cuasr/gemm/kernel/srgemm.h:156-321
// with DefaultSemiRingConfiguration<plus, multiplies>,
// include/cuasr/gemm/device/default_srgemm_configuration.h:44-72).  The sum over
// k is formed in the instruction's order (pairs of k, fused multiply-adds), not
// the host reference's strictly sequential unfused order, so results agree with
// it to rounding -- |d - r| <= 1e-5 * sum_k |a||b| -- not bit for bit; the
// vector-ALU tile (kernel = VALU / VALU_DIRECT) stays available for a bit-exact
// plus-times.
//
// Workgroup 256 threads = 4 waves (2 x 2), output tile 128 x 128, wave tile
// 64 x 64 = 2 x 2 blocks of 32 x 32 (64 accumulator registers), k-tile 16; or
// output tile 128 x 256, wave tile 64 x 128 (128 accumulator registers).
// LDS per stage: A and B k-major, [k][LD] floats.  The instruction wants k = 2q
// from lanes 0..31 and k = 2q + 1 from lanes 32..63, each lane one float of
// its row: 32 consecutive floats of LDS row 2q and 32 of row 2q + 1 per read,
// which no bank layout can make collide.  LD = 160 puts consecutive rows 32
// banks apart; rows of odd k-quads have bit 4 of the column flipped so that
// the four k-quads a wave writes at once (k-contiguous operands: 16 rows x 4
// quads per wave) spread over all banks instead of piling onto 16 of them.
#include "mfma_common.h"

namespace cuasr_amd {

bool mfma_direct_f32_can_run(const Problem &);                // mfma_direct_f32.hip
hipError_t mfma_direct_f32_launch(const Problem &, bool wide, hipStream_t);

namespace gemm_mfma {

using namespace mfma_panel;

constexpr int LD = 160;
__device__ __forceinline__ int swz(int k) { return ((k >> 2) & 1) << 4; }

// NB: 128-column halves of the B panel.  1: output tile 128 x 128, wave tile 64 x 64.  2: output
// tile 128 x 256, wave tile 64 x 128 -- six LDS reads per sixteen matrix instructions instead of
// four per eight, and a quarter less global traffic per flop; for outputs that fill its rounds.
template <int NB> struct Smem {
  float a[2][BK][LD];
  float b[2][NB][BK][LD];
};

// One operand's share of a thread in the global -> LDS copy of a 128 x 16 panel:
// two 16-byte vectors.
//   x contiguous: vector j = 4 consecutive x at one k
//   k contiguous: vector q = 4 consecutive k at one x
// src[] points at the vectors of the FIRST k-tile (x clamped to the matrix) and
// advances by `step` per tile; lds[] is the float index inside a stage where
// element 0 of each vector goes (row stride LD per k for k-contiguous vectors).
// LOOSE: operands of any extent, leading dimension and 4-byte alignment.  The vector loads are made at element
// alignment (the hardware takes them at any 4-byte boundary), and a vector that would cross the end of its row
// (x contiguous) or of the k range (k contiguous) is read element by element with clamped indices instead --
// what lands in the places past the end is never used (rows / columns past the edge are not stored, k past the
// end is zeroed in the ragged tile).
typedef float v4f_loose __attribute__((ext_vector_type(4), aligned(4)));

template <bool LOOSE> struct Mover {
  const float *src[2];
  long long step;
  int lds[2];
  bool x_contig;
  int x_left;    // LOOSE, x contiguous: elements from this thread's vector start to the end of the row (<= 0: none)

  __device__ __forceinline__ void init(const float *base, long long s_x, long long s_k, int x0, int x_end, int k0,
                                       bool xc) {
    const int tid = threadIdx.x;
    x_contig = xc;
    step = (long long)BK * s_k;
    if (xc) {
      const int xg = tid & 31, kq = (tid >> 5) & 3, half = tid >> 7;
      const int xx = LOOSE ? min(x0 + xg * 4, x_end - 1) : min(x0 + xg * 4, x_end - 4);
      x_left = x_end - (x0 + xg * 4);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int kk = kq * 4 + half * 2 + j;
        src[j] = base + (long long)(k0 + kk) * s_k + xx;
        lds[j] = kk * LD + ((xg * 4) ^ swz(kk));
      }
    } else {
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        // lanes 0..15: 16 consecutive x of k-quad 0, lanes 16..31: the same x of k-quad 1, ...
        const int f = tid + 256 * q;
        const int x = ((f >> 6) << 4) | (f & 15), kg = (f >> 4) & 3;
        const int xx = min(x0 + x, x_end - 1);
        src[q] = base + (long long)xx * s_x + k0 + kg * 4;
        lds[q] = kg * 4 * LD + (x ^ swz(kg * 4));
      }
    }
  }
  // 4 consecutive x from `at`, of which x_left lie inside the row (LOOSE; at itself is inside)
  __device__ __forceinline__ v4f row_vector(const float *at) const {
    if (x_left >= 4) return *reinterpret_cast<const v4f_loose *>(at);
    v4f v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = at[min(e, max(x_left - 1, 0))];
    return v;
  }
  // whole k-tile: nothing to clamp along k
  __device__ __forceinline__ void load(v4f (&r)[2]) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (!LOOSE) r[j] = *reinterpret_cast<const v4f *>(src[j]);
      else if (x_contig) r[j] = row_vector(src[j]);
      else r[j] = *reinterpret_cast<const v4f_loose *>(src[j]);
    }
  }
  // ragged last k-tile with `kcount` (< BK) valid k: vectors that start past the end re-read the
  // last valid one (never used); k-contiguous extents are multiples of 4, so no vector straddles the end
  __device__ __forceinline__ void load_ragged(v4f (&r)[2], long long s_k, int kcount) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      long long back = 0;
      if (x_contig) {
        const int kk = ((tid >> 5) & 3) * 4 + (tid >> 7) * 2 + j;
        back = (long long)max(kk - (kcount - 1), 0) * s_k;
        if constexpr (LOOSE) {
          r[j] = row_vector(src[j] - back);
          continue;
        }
      } else {
        const int kg = ((tid + 256 * j) >> 4) & 3;
        if constexpr (LOOSE) {
          // element e is k = 4 kg + e of the tile; past the end, the last valid k instead
          if (kg * 4 + 4 <= kcount) {
            r[j] = *reinterpret_cast<const v4f_loose *>(src[j]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) r[j][e] = src[j][min(kg * 4 + e, kcount - 1) - kg * 4];
          }
          continue;
        }
        back = max(kg * 4 - (kcount - 4), 0);
      }
      r[j] = *reinterpret_cast<const v4f *>(src[j] - back);
    }
  }
  __device__ __forceinline__ void advance() {
    src[0] += step;
    src[1] += step;
  }
  __device__ __forceinline__ void store(const v4f (&r)[2], float *stage) const {
    if (x_contig) {
#pragma unroll
      for (int j = 0; j < 2; ++j) *reinterpret_cast<v4f *>(stage + lds[j]) = r[j];
    } else {
#pragma unroll
      for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) stage[lds[q] + e * LD] = r[q][e];
    }
  }
};

template <int NB, bool LOOSE = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_mfma_kernel(Problem p) {
  constexpr int BN = 128 * NB, WN = 64 * NB, QB = 2 * NB;  // tile columns, wave columns, 32-column blocks per wave
  __shared__ Smem<NB> sm;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  int bm, bn;
  tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
  const int m0 = bm * BM, n0 = bn * BN;
  const float *A = reinterpret_cast<const float *>(p.A);
  const float *B = reinterpret_cast<const float *>(p.B);

  int kb = 0, ke = p.k;
  if (p.workspace) {
    kb = blockIdx.y * p.k_per_slice;
    ke = min(p.k, kb + p.k_per_slice);
  }
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;

  // byte offset, inside the LDS panel array, of this lane's operand for k-pair 0 of an even / odd k-quad
  int a_idx[2][2], b_idx[QB][2];
#pragma unroll
  for (int o = 0; o < 2; ++o) {
#pragma unroll
    for (int q = 0; q < 2; ++q) a_idx[q][o] = 4 * ((lane >> 5) * LD + ((wm * 64 + q * 32 + (lane & 31)) ^ (o << 4)));
#pragma unroll
    for (int q = 0; q < QB; ++q) {
      const int c = wn * WN + q * 32;  // the block's first column inside the tile: half c / 128, column c % 128 of it
      b_idx[q][o] = 4 * ((c >> 7) * BK * LD + (lane >> 5) * LD + (((c & 127) + (lane & 31)) ^ (o << 4)));
    }
  }

  v16f acc[2][QB];
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < QB; ++bj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bi][bj][r] = p.add_identity.f32;  // 0 for plus

  const int ntiles = (ke - kb + BK - 1) / BK;
  Mover<LOOSE> ma, mb[NB];
  ma.init(A, p.sa_m, p.sa_k, m0, p.m, kb, a_xc);
#pragma unroll
  for (int h = 0; h < NB; ++h) mb[h].init(B, p.sb_n, p.sb_k, n0 + 128 * h, p.n, kb, b_xc);
  v4f ra[2], rb[NB][2];
  // k-tile t into registers; `whole` says at compile time whether it has all BK values of k
  // (one code path per call site: merged paths made the compiler wait for the first three loads
  // of a tile before issuing the fourth)
  auto fetch = [&](int t, auto whole) {
    if constexpr (decltype(whole)::value) {
      ma.load(ra);
#pragma unroll
      for (int h = 0; h < NB; ++h) mb[h].load(rb[h]);
    } else {
      const int kcount = ke - (kb + t * BK);
      ma.load_ragged(ra, p.sa_k, kcount);
#pragma unroll
      for (int h = 0; h < NB; ++h) mb[h].load_ragged(rb[h], p.sb_k, kcount);
    }
    ma.advance();
#pragma unroll
    for (int h = 0; h < NB; ++h) mb[h].advance();
  };
  auto store = [&](int stage) {
    ma.store(ra, &sm.a[stage][0][0]);
#pragma unroll
    for (int h = 0; h < NB; ++h) mb[h].store(rb[h], &sm.b[stage][h][0][0]);
  };
  const int nfull = max(ke - kb, 0) / BK;
  if (ntiles > 0) {
    if (nfull > 0) fetch(0, std::true_type{});
    else fetch(0, std::false_type{});
    store(0);
  }
  __syncthreads();

  int buf = 0, a_step = BK * LD * 4, b_step = NB * BK * LD * 4;
  constexpr int STORE_AT = KQ - 2;
  // One k-tile: the next tile's global loads, this tile's matrix instructions, the next tile's
  // LDS stores, a barrier.  RAGGED (the last tile of a k range that is not a multiple of BK): k
  // past the end must not count.  The panels hold other (finite or not) data there, so the
  // operands of those k are replaced by zeros: 0 * 0 adds nothing.  Kept out of the steady-state
  // loop, whose body then has no branch (125.6 -> 130.3 TFLOP/s at 4096^3).  Order inside a tile:
  // the next tile's global loads first, its LDS stores after the third of the four k-quads, so
  // that they run under the last quad's matrix instructions instead of between them and the
  // barrier (2048^3: 88.6 -> 110.3 TFLOP/s, 6144^3: 117.7 -> 127.7); the LDS reads stay where the
  // compiler puts them -- a k-quad ahead of their use measured slower (114 TFLOP/s at 4096^3).
  // NEXT: what follows this tile -- 2 a whole tile, 1 a ragged one, 0 nothing
  auto tile = [&](int t, auto ragged, auto next) {
    constexpr bool RAGGED = decltype(ragged)::value;
    constexpr int NEXT = decltype(next)::value;
    constexpr bool more = NEXT != 0;
    if constexpr (NEXT == 2) fetch(t + 1, std::true_type{});
    if constexpr (NEXT == 1) fetch(t + 1, std::false_type{});
    __builtin_amdgcn_sched_barrier(0);
    const int kcount = ke - (kb + t * BK);
    const char *pa = reinterpret_cast<const char *>(&sm.a[0][0][0]);
    const char *pb = reinterpret_cast<const char *>(&sm.b[0][0][0][0]);
#pragma unroll
    for (int kq = 0; kq < KQ; ++kq) {
      float av[2][2], bv[QB][2];  // [block][k-pair of the quad]
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int q = 0; q < 2; ++q) av[q][j] = *reinterpret_cast<const float *>(pa + (kq * 4 + 2 * j) * LD * 4 + a_idx[q][kq & 1]);
#pragma unroll
        for (int q = 0; q < QB; ++q) bv[q][j] = *reinterpret_cast<const float *>(pb + (kq * 4 + 2 * j) * LD * 4 + b_idx[q][kq & 1]);
      }
      if constexpr (RAGGED) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const bool valid = kq * 4 + 2 * j + (lane >> 5) < kcount;
#pragma unroll
          for (int q = 0; q < 2; ++q) av[q][j] = valid ? av[q][j] : 0.0f;
#pragma unroll
          for (int q = 0; q < QB; ++q) bv[q][j] = valid ? bv[q][j] : 0.0f;
        }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int bi = 0; bi < 2; ++bi)
#pragma unroll
          for (int bj = 0; bj < QB; ++bj)
            acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[bi][j], bv[bj][j], acc[bi][bj], 0, 0, 0);
      if (kq == STORE_AT) {
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (more) store(buf ^ 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
    buf ^= 1;
    // the lane's read indices follow the stage: one add each instead of an address per read
#pragma unroll
    for (int o = 0; o < 2; ++o) {
#pragma unroll
      for (int q = 0; q < 2; ++q) a_idx[q][o] += a_step;
#pragma unroll
      for (int q = 0; q < QB; ++q) b_idx[q][o] += b_step;
    }
    a_step = -a_step;
    b_step = -b_step;
  };
  using whole_next = std::integral_constant<int, 2>;
  using ragged_next = std::integral_constant<int, 1>;
  using no_next = std::integral_constant<int, 0>;
  for (int t = 0; t + 1 < nfull; ++t) tile(t, std::false_type{}, whole_next{});
  if (nfull > 0) {
    if (nfull < ntiles) tile(nfull - 1, std::false_type{}, ragged_next{});
    else tile(nfull - 1, std::false_type{}, no_next{});
  }
  if (nfull < ntiles) tile(nfull, std::true_type{}, no_next{});

  // ---- epilogue.  Block (bi, bj), register r of lane l holds
  // row = 8*(r/4) + 4*(l/32) + r%4, column = l%32 of the 32 x 32 block.
  float *out;
  long long ld_out;
  const bool partial = p.workspace != nullptr;
  float alpha = 1.f, beta = 0.f;
  bool source_needed = false;
  if (partial) {
    out = reinterpret_cast<float *>(p.workspace) + (long long)blockIdx.y * p.m * p.n;
    ld_out = p.n;
  } else {
    out = reinterpret_cast<float *>(p.D);
    ld_out = p.ldd;
    const EpilogueScalars<float> e = resolve_scalars<float>(p, kMultiplies);
    alpha = e.alpha;
    beta = e.beta;
    source_needed = e.source_needed;
  }
  const float *C = reinterpret_cast<const float *>(p.C);
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < QB; ++bj) {
      const int col = n0 + wn * WN + bj * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * 64 + bi * 32 + 8 * (r / 4) + 4 * (lane >> 5) + (r % 4);
        if (row < p.m && col < p.n) {
          float v = acc[bi][bj][r];
          if (!partial) {
            v = alpha * v;
            if (source_needed) v = v + beta * C[(long long)row * p.ldc + col];
          }
          out[(long long)row * ld_out + col] = v;
        }
      }
    }
}

static hipError_t launch(const Problem &p, hipStream_t s) {
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!loose_can_run(p)) return hipErrorNotSupported;
  const bool loose = !can_run(p);
  const long long tiles_m = (p.m + BM - 1) / BM, slices = p.workspace ? p.slices : 1;
  const long long tiles = tiles_m * ((p.n + 127) / 128), wide = tiles_m * ((p.n + 255) / 256);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  // Whole k-tiles and loadable straight into LDS: the hand-scheduled forms of the two tiles.  A compute unit's
  // matrix pipes are as busy with one workgroup as with three, so a launch takes about ceil(tiles / 256) tile
  // times, and the tile that wastes less of its last such round wins (2048^3: 132 against 71 TFLOP/s for the narrow
  // tile, 5120^3: 133 against 117, 6144^3: 150 against 136); where both fill theirs (4096^3: 149.1 and 149.8) the
  // wide one, which moves a quarter less data per flop.
  const long long batch = p.batch > 1 ? p.batch : 1;
  if (!loose && mfma_direct_f32_can_run(p)) {
    auto fill = [](long long groups) { return (double)groups / (256.0 * (double)((groups + 255) / 256)); };
    return mfma_direct_f32_launch(p, fill(wide * slices * batch) >= 0.995 * fill(tiles * slices * batch), s);
  }
  if (batch > 1) return hipErrorNotSupported;  // the compiled kernels take one product per launch
  // the 128 x 256 tile when its workgroups fill >= 7/8 of whole rounds of 512 (two per compute unit)
  const long long rounds = (wide * slices + 511) / 512;
  const bool wide_tile = wide * slices * 8 >= rounds * 512 * 7;
  const dim3 grid((unsigned)(wide_tile ? wide : tiles), (unsigned)slices);
  if (loose) {
    if (wide_tile) launch_kernel((gemm_mfma_kernel<2, true>), grid, dim3(256), 0, s, p);
    else launch_kernel((gemm_mfma_kernel<1, true>), grid, dim3(256), 0, s, p);
  } else {
    if (wide_tile) launch_kernel((gemm_mfma_kernel<2, false>), grid, dim3(256), 0, s, p);
    else launch_kernel((gemm_mfma_kernel<1, false>), grid, dim3(256), 0, s, p);
  }
  return take_launch_status();
}

}  // namespace gemm_mfma

// plus-times runs on the matrix cores whatever the operands' extents and alignment
bool mfma_gemm_f32_can_run(const Problem &p) { return mfma_panel::loose_can_run(p); }

launch_fn find_mfma_gemm_f32(int add_op, int mult_op) {
  if (add_op == kPlus && mult_op == kMultiplies) return gemm_mfma::launch;
  return nullptr;
}

}  // namespace cuasr_amd
