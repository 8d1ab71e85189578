// Direct-to-LDS vector-ALU SRGEMM tile for 8-byte element types on gfx950.
//
// Same role as direct_tile.h (in the reference: threadblock/srmma_pipelined.h:153-288,
// warp/srmma_simt.h:190-199, thread/srmma_sm50.h:118-146, kernel/srgemm.h:156-321).  fp64 vector
// instructions issue at 16 lanes per clock and there is no 3-input fp64 min/max, so a term costs two
// instructions whatever the tile; what the tile can add is occupancy: an fp64 instruction issues every
// ~4.5 cycles per SIMD at 4 waves, 4.6 at 3, 4.9 at 2 (LDS reads, waits and scalar instructions hide
// beneath them).  Panels go global -> LDS without passing through registers, and the main loop is
// hand-scheduled asm (direct_asm.h): accumulators (64 registers), ONE set of fragments of a k-pair (48)
// refilled in place and four temporaries stay inside 128 registers = 4 waves per SIMD.
//
//   workgroup 512 threads (16 x 32), output tile 128 x 128, thread tile 8 x 4, k-tile 16,
//   two LDS stages (64 KiB; two workgroups per compute unit = 16 waves).
//
// LDS forms (the image equals the lane fetch order of the 16-byte loads), X = 128 for both panels:
//   x-contiguous operand: [k][X]       one 16-byte read = 2 x at one k
//   k-contiguous operand: [k/2][X][2]  one 16-byte read = both k of a pair at one x
// Thread t of XT along a panel owns, of its 8 (A) or 4 (B) rows / columns,
//   x-contiguous: x = (i / 2) * 2 XT + 2 t + i % 2        k-contiguous: x = XT * i + t.
// Needs 16-byte aligned operands with even leading dimensions and extents
// (see direct64_ok); everything else goes to the staged tile.
#pragma once
#include <utility>
#include "direct_asm.h"
#include "semiring.h"

namespace cuasr_amd {

// what the tile shares with nothing else: the global -> LDS addressing and the tile order
struct Direct64Base {
  // A panel's LDS image has X * 16 / 2 positions of 16 bytes; a position's global address is
  // (uniform base of this k-tile) + (per-lane byte offset, 32 bits: the host checks that a tile
  // spans less than 2 GiB).  Indices past the matrix edge or past the last valid k of a ragged
  // tile are clamped to the last valid vector (never used).
  template <bool KC, int X>
  static __device__ __forceinline__ unsigned tile_offset(int pos, long long s_x, unsigned s_k_bytes, int x0, int x_end, int kcount) {
    if constexpr (KC) {
      const int x = min(x0 + pos % X, x_end - 1) - x0, k = min((pos / X) * 2, kcount - 2);
      return (unsigned)x * (unsigned)s_x * 8u + (unsigned)k * 8u;
    } else {
      const int x = min(x0 + (pos % (X / 2)) * 2, x_end - 2) - x0, k = min(pos / (X / 2), kcount - 1);
      return (unsigned)x * 8u + (unsigned)k * s_k_bytes;
    }
  }
  template <typename T> static __device__ __forceinline__ void dma16(const char *src, T *lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                     (__attribute__((address_space(3))) void *)lds_wave_base, 16, 0, 0);
  }
  static __device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int &bm, int &bn) {
    const int total = tiles_m * tiles_n;
    // consecutive workgroup ids land on consecutive XCDs (8, one L2 each):
    // give every XCD one contiguous run of the tile order
    if ((total & 7) == 0) id = (id & 7) * (total >> 3) + (id >> 3);
    constexpr int GROUP = 8;
    const int width = GROUP * tiles_n;
    const int group = id / width, first = group * GROUP;
    const int gsz = min(tiles_m - first, GROUP);
    bm = first + (id % width) % gsz;
    bn = (id % width) / gsz;
  }
};

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC>
struct Direct64Tile {
  static_assert(sizeof(T) == 8, "8-byte element types only");
  typedef Direct64Base Base;
  typedef typename AsmLoop<T, ADD, MUL, A_KC, B_KC>::type Loop;
  static constexpr int TY = 16, TX = 32, BM = 8 * TY, BN = 4 * TX, BK = 16, THREADS = TY * TX, WAVES = THREADS / 64, STAGES = 2;
  static constexpr int LA = BM * BK * 8 / 1024 / WAVES, LB = BN * BK * 8 / 1024 / WAVES;  // 2, 2
  static_assert(LA == 2 && LB == 2, "the generated loop moves two pieces of each panel per wave");
  typedef T vec2 __attribute__((ext_vector_type(2)));

  struct Smem {
    T a[STAGES][BK * BM];
    T b[STAGES][BK * BN];
  };

  template <bool KC, int XT> static __device__ __forceinline__ int own(int i, int t) {
    return KC ? i * XT + t : (i >> 1) * 2 * XT + t * 2 + (i & 1);
  }
  template <bool KC, int N, int XT> static __device__ __forceinline__ void load_frag1(T (&f)[N], const T *panel, int kk, int t) {
    constexpr int X = N * XT;
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int x = own<KC, XT>(i, t);
      f[i] = KC ? panel[((kk >> 1) * X + x) * 2 + (kk & 1)] : panel[kk * X + x];
    }
  }

  static __device__ __forceinline__ void run(const Problem &p, Smem &sm) {
    const int tid = threadIdx.x, tx = tid % TX, ty = tid / TX, lane = tid & 63, wave = tid >> 6;
    const int tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
    int bm, bn;
    Base::tile_coords(blockIdx.x, tiles_m, tiles_n, bm, bn);
    const int m0 = bm * BM, n0 = bn * BN;
    const T *A = reinterpret_cast<const T *>(p.A);
    const T *B = reinterpret_cast<const T *>(p.B);
    const T ident = scalar_as<T>(p.add_identity);

    int kb = 0, ke = p.k;
    if (p.workspace) {
      kb = blockIdx.y * p.k_per_slice;
      ke = min(p.k, kb + p.k_per_slice);
    }

    const char *base_a = reinterpret_cast<const char *>(A + (long long)m0 * p.sa_m + (long long)kb * p.sa_k);
    const char *base_b = reinterpret_cast<const char *>(B + (long long)n0 * p.sb_n + (long long)kb * p.sb_k);
    const long long a_step = (long long)BK * p.sa_k * 8, b_step = (long long)BK * p.sb_k * 8;
    const unsigned a_kbytes = (unsigned)p.sa_k * 8u, b_kbytes = (unsigned)p.sb_k * 8u;
    auto off_a = [&](int q, int kcount) { return Base::template tile_offset<A_KC, BM>((wave * LA + q) * 64 + lane, p.sa_m, a_kbytes, m0, p.m, kcount); };
    auto off_b = [&](int q, int kcount) { return Base::template tile_offset<B_KC, BN>((wave * LB + q) * 64 + lane, p.sb_n, b_kbytes, n0, p.n, kcount); };
    // k-tile with kcount valid k into an LDS stage (compiler-issued: prologue and a ragged last tile)
    auto fetch = [&](int stage, int kcount) {
      if (kcount > 0) {
#pragma unroll
        for (int q = 0; q < LA; ++q) Base::dma16<T>(base_a + off_a(q, kcount), &sm.a[stage][(wave * LA + q) * 128]);
#pragma unroll
        for (int q = 0; q < LB; ++q) Base::dma16<T>(base_b + off_b(q, kcount), &sm.b[stage][(wave * LB + q) * 128]);
      }
    };

    const int nfull = (ke - kb) / BK, rem = (ke - kb) - nfull * BK;  // whole k-tiles, then one ragged tile
    auto tile_k = [&](int t) { return t < nfull ? BK : (t == nfull ? rem : 0); };
    fetch(0, tile_k(0));
    base_a += a_step;
    base_b += b_step;
    __syncthreads();
    fetch(1, tile_k(1));
    base_a += a_step;
    base_b += b_step;  // base_a / base_b now point at tile 2

    T acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = ident;

    if (nfull > 0) {
      AsmRegs r;
      const unsigned long long ident_bits = __builtin_bit_cast(unsigned long long, ident);
      const float ident_lo = __builtin_bit_cast(float, (unsigned)ident_bits), ident_hi = __builtin_bit_cast(float, (unsigned)(ident_bits >> 32));
#pragma unroll
      for (int v = 0; v < 4; ++v)
#pragma unroll
        for (int e = 0; e < 16; ++e) r.acc[v][e] = (e & 1) ? ident_hi : ident_lo;
#pragma unroll
      for (int v = 0; v < 3; ++v) r.frag[v] = asm_v16(0.0f);
      const unsigned oa0 = off_a(0, BK), oa1 = off_a(1, BK), ob0 = off_b(0, BK), ob1 = off_b(1, BK);
      // LDS byte address of this wave's first piece of each panel in stage 0 (wave-uniform)
      const unsigned m0_a0 = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.a[0][(wave * LA) * 128]);
      const unsigned m0_b0 = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.b[0][(wave * LB) * 128]);
      constexpr unsigned A_STAGE = BK * BM * 8, B_STAGE = BK * BN * 8;
      unsigned a_addr = (unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.a[0][0] + ty * 16;
      unsigned b_addr = (unsigned)(size_t)(__attribute__((address_space(3))) T *)&sm.b[0][0] + tx * 16;
      Loop::prime(r, a_addr, b_addr);
      for (int t = 0; t < nfull; ++t) {
        const int stage = t & 1;
        // the statement's barrier hands stage `stage` back; the tile two ahead goes there: a whole one
        // from inside the statement, a ragged one from here right after it
        Loop::tile(r, a_addr, b_addr, stage ? 0u - A_STAGE : A_STAGE, stage ? 0u - B_STAGE : B_STAGE, nfull - (t + 2),
                   m0_a0 + stage * A_STAGE, m0_b0 + stage * B_STAGE, oa0, oa1, ob0, ob1, base_a, base_b);
        if (t + 2 == nfull) fetch(stage, rem);
        base_a += a_step;
        base_b += b_step;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const unsigned lo = __builtin_bit_cast(unsigned, (float)r.acc[i >> 1][(i & 1) * 8 + 2 * j]);
          const unsigned hi = __builtin_bit_cast(unsigned, (float)r.acc[i >> 1][(i & 1) * 8 + 2 * j + 1]);
          acc[i][j] = __builtin_bit_cast(T, ((unsigned long long)hi << 32) | lo);
        }
    }
    if (rem > 0) {
      if (nfull == 0) __syncthreads();  // (with whole tiles before it, the last statement's barrier covers the ragged tile)
      const int buf = nfull & 1;
      const T *pa = sm.a[buf], *pb = sm.b[buf];
#pragma unroll 1
      for (int kk = 0; kk < rem; ++kk) {
        T fa[8], fb[4];
        load_frag1<A_KC, 8, TY>(fa, pa, kk, ty);
        load_frag1<B_KC, 4, TX>(fb, pb, kk, tx);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = fold<ADD, MUL>(Op<MUL>::apply(fa[i], fb[j]), acc[i][j]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }

    // ---- epilogue: D = add(mult(alpha, acc), mult(beta, C)), or raw partials
    T *out;
    long long ld_out;
    const bool partial = p.workspace != nullptr;
    EpilogueScalars<T> e;
    if (partial) {
      out = reinterpret_cast<T *>(p.workspace) + (long long)blockIdx.y * p.m * p.n;
      ld_out = p.n;
      e.alpha = e.beta = e.ident = ident;
      e.source_needed = false;
    } else {
      out = reinterpret_cast<T *>(p.D);
      ld_out = p.ldd;
      e = resolve_scalars<T>(p, MUL);
    }
    const T *C = reinterpret_cast<const T *>(p.C);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = m0 + own<A_KC, TY>(i, ty);
      if ((unsigned)row < (unsigned)p.m) {
        if constexpr (!B_KC) {
#pragma unroll
          for (int g = 0; g < 2; ++g) {
            const int col = n0 + g * 2 * TX + tx * 2;
            if ((unsigned)col < (unsigned)p.n) {  // n is even here: the pair is inside
              vec2 v = {acc[i][2 * g], acc[i][2 * g + 1]};
              if (!partial) {
#pragma unroll
                for (int c = 0; c < 2; ++c) v[c] = Op<MUL>::apply(e.alpha, v[c]);
                if (e.source_needed) {
                  const vec2 s = *reinterpret_cast<const vec2 *>(C + (long long)row * p.ldc + col);
#pragma unroll
                  for (int c = 0; c < 2; ++c) v[c] = fold_epilogue<ADD, MUL>(v[c], Op<MUL>::apply(e.beta, s[c]));
                }
              }
              *reinterpret_cast<vec2 *>(out + (long long)row * ld_out + col) = v;
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int col = n0 + own<true, TX>(j, tx);
            if ((unsigned)col < (unsigned)p.n) {
              T v = acc[i][j];
              if (!partial) {
                v = Op<MUL>::apply(e.alpha, v);
                if (e.source_needed) v = fold_epilogue<ADD, MUL>(v, Op<MUL>::apply(e.beta, C[(long long)row * p.ldc + col]));
              }
              out[(long long)row * ld_out + col] = v;
            }
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

template <typename T, int ADD, int MUL, bool A_KC, bool B_KC>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void direct64_srgemm_kernel(Problem p) {
  using Tile = Direct64Tile<T, ADD, MUL, A_KC, B_KC>;
  __shared__ typename Tile::Smem sm;
  select_batch<T>(p);
  Tile::run(p, sm);
}

// can the fp64 direct tile run this (canonical) problem?
static inline bool direct64_ok(const Problem &p) {
  auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  if (p.k <= 0 || !al(p.A) || !al(p.B)) return false;
  // every product of a batch in the grid starts at base + index * stride: the strides keep the 16-byte alignment
  if (p.batch > 1 && ((p.batch_a | p.batch_b | p.batch_c | p.batch_d) % 2)) return false;
  // 32-bit byte offsets inside one tile
  const long long span = 8LL * 128 * (p.sa_m > p.sa_k ? p.sa_m : p.sa_k), span_b = 8LL * 128 * (p.sb_n > p.sb_k ? p.sb_n : p.sb_k);
  if (span >= (1LL << 31) || span_b >= (1LL << 31)) return false;
  if (a_kc ? (p.k % 2 || p.sa_m % 2) : (p.sa_m != 1 || p.m % 2 || p.sa_k % 2)) return false;
  if (b_kc ? (p.k % 2 || p.sb_n % 2) : (p.sb_n != 1 || p.n % 2 || p.sb_k % 2)) return false;
  if (!b_kc) {  // 16-byte stores of D (and loads of C)
    if (p.n % 2) return false;
    if (p.workspace) {
      if (!al(p.workspace)) return false;
    } else {
      if (!al(p.D) || p.ldd % 2) return false;
      if (p.C && (!al(p.C) || p.ldc % 2)) return false;
    }
  }
  return true;
}

template <typename T, int ADD, int MUL> static hipError_t launch_direct64(const Problem &p, hipStream_t s) {
  static_assert(!std::is_void<typename AsmLoop<T, ADD, MUL, false, false>::type>::value, "no main loop for this semiring");
  if (p.m == 0 || p.n == 0) return hipSuccess;
  if (!direct64_ok(p)) return hipErrorNotSupported;
  const long long tiles = (long long)((p.m + 127) / 128) * ((p.n + 127) / 128);
  if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, p.workspace ? p.slices : 1, p.batch);
  const bool a_kc = p.sa_k == 1 && p.sa_m != 1, b_kc = p.sb_k == 1 && p.sb_n != 1;
  if (a_kc && b_kc) launch_kernel((direct64_srgemm_kernel<T, ADD, MUL, true, true>), grid, dim3(512), 0, s, p);
  else if (a_kc) launch_kernel((direct64_srgemm_kernel<T, ADD, MUL, true, false>), grid, dim3(512), 0, s, p);
  else if (b_kc) launch_kernel((direct64_srgemm_kernel<T, ADD, MUL, false, true>), grid, dim3(512), 0, s, p);
  else launch_kernel((direct64_srgemm_kernel<T, ADD, MUL, false, false>), grid, dim3(512), 0, s, p);
  return take_launch_status();
}

}  // namespace cuasr_amd
