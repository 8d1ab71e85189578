// Pieces shared by the matrix-core tiles for float: vector types, the
// global -> register -> LDS staging of a 128 x 16 panel in the [k/4][row][4]
// form (4 consecutive k of one row per 16 bytes), the workgroup -> tile
// mapping and the operand requirements.
#pragma once
#include "semiring.h"

namespace cuasr_amd {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

namespace mfma_panel {

constexpr int BM = 128, BN = 128, BK = 16, KQ = BK / 4;

// Global -> registers for one 128 x 16 panel (8 floats per thread).
//   k contiguous: two 16-byte loads, each 4 consecutive k of one row
//   x contiguous: two 16-byte loads, each 4 consecutive rows at one k
// Out-of-range rows / k are clamped to the last valid vector (never used).
__device__ __forceinline__ void load_panel(v4f (&r)[2], const float *base, long long s_x, long long s_k, int x0,
                                           int x_end, int k0, int k_end, bool x_contig) {
  const int tid = threadIdx.x;
  if (x_contig) {
    const int xg = tid & 31, kq = (tid >> 5) & 3, half = tid >> 7;
    const int xx = min(x0 + xg * 4, x_end - 4);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int kk = min(k0 + kq * 4 + half * 2 + j, k_end - 1);
      r[j] = *reinterpret_cast<const v4f *>(base + (long long)kk * s_k + xx);
    }
  } else {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int f = tid + 256 * q;
      const int xx = min(x0 + (f >> 2), x_end - 1);
      const int kk = min(k0 + (f & 3) * 4, k_end - 4);
      r[q] = *reinterpret_cast<const v4f *>(base + (long long)xx * s_x + kk);
    }
  }
}

template <int ROWS>
__device__ __forceinline__ void store_panel(const v4f (&r)[2], v4f (*dst)[ROWS], bool x_contig) {
  const int tid = threadIdx.x;
  if (x_contig) {
    const int xg = tid & 31, kq = (tid >> 5) & 3, half = tid >> 7;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v2f t = {r[0][e], r[1][e]};
      *reinterpret_cast<v2f *>(reinterpret_cast<float *>(&dst[kq][xg * 4 + e]) + half * 2) = t;
    }
  } else {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int f = tid + 256 * q;
      dst[f & 3][f >> 2] = r[q];
    }
  }
}

__device__ __forceinline__ void tile_coords(int id, int tiles_m, int tiles_n, int &bm, int &bn) {
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

// the loads are 16-byte vectors: aligned bases, leading dimensions that are
// multiples of 4 and extents of at least one vector along the contiguous
// direction (so a clamped vector stays inside the matrix)
static inline bool can_run(const Problem &p) {
  auto al = [](const void *q) { return reinterpret_cast<uintptr_t>(q) % 16 == 0; };
  const bool a_xc = p.sa_m == 1, b_xc = p.sb_n == 1;
  if (!al(p.A) || !al(p.B)) return false;
  if (a_xc ? (p.m % 4 || p.sa_k % 4) : (p.sa_k != 1 || p.k % 4 || p.sa_m % 4)) return false;
  if (b_xc ? (p.n % 4 || p.sb_k % 4) : (p.sb_k != 1 || p.k % 4 || p.sb_n % 4)) return false;
  return true;
}

// what the element-aligned form of the compiled plus-times kernel asks for: one contiguous direction per operand
static inline bool loose_can_run(const Problem &p) {
  return (p.sa_m == 1 || p.sa_k == 1) && (p.sb_n == 1 || p.sb_k == 1);
}

}  // namespace mfma_panel
}  // namespace cuasr_amd
