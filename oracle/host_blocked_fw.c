/*
 * CPU oracle for blocked Floyd-Warshall with predecessor tracking -- TEST
 * INFRASTRUCTURE ONLY (see host_srgemm.c: only tests/, smoke() and the
 * cpu_baseline leg of bench.py may use this library).
 *
 * The reference has no blocked Floyd-Warshall; its README names all-pairs
 * shortest paths as the application (README.md:338-342) and its legacy code
 * holds the building block, the min-plus product that records the k of every
 * strict improvement (cpu_fwgemm_naive,
 * test/regress/include/fwgpu/cpu_srgemm.hpp:20-48).  This file states the
 * blocked algorithm built from that block, in the order of operations the
 * device driver uses, so that the two can be compared bit for bit:
 *
 *   for every diagonal block [k0, k0 + b):
 *     1. Floyd-Warshall inside the block, in place: k ascending,
 *        d[i][j] > d[i][k] + d[k][j]  =>  d[i][j] = that sum, parent = k0 + k;
 *     2. R = copy of block row k0 (b x n), C = copy of block column k0 (n x b);
 *     3. block row    <- fwgemm(R[:, k0:k0+b], R)   (parents offset by k0),
 *        block column <- fwgemm(C, C[k0:k0+b, :]),
 *        both leaving the diagonal block, which is closed, as it is;
 *     4. every element outside block row and block column k0
 *                     <- fwgemm(block column, block row).
 *
 * Parity status: pinned by tests/test_oracle.py -- distances against scipy's
 * Floyd-Warshall and against the literal triple loop on integer weights (where
 * every order of additions is exact), for several block sizes and ragged n;
 * parents by rebuilding paths whose edge weights sum to the distance; a
 * hand-worked graph.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define DEFINE_BLOCKED_FW(NAME, T)                                                          \
  /* the product of cpu_fwgemm_naive with parents offset by k_base; elements in the rows    \
     [sr0, sr1) or the columns [sc0, sc1) are left alone */                                  \
  static void NAME##_product(int m, int n, int k, const T *A, int64_t lda, const T *B,      \
                             int64_t ldb, T *dist, int64_t ldc, int32_t *parent,             \
                             int64_t ldp, int k_base, int sr0, int sr1, int sc0, int sc1) {  \
    _Pragma("omp parallel for schedule(static)")                                            \
    for (int col = 0; col < n; ++col) {                                                     \
      if (col >= sc0 && col < sc1) continue;                                                \
      for (int row = 0; row < m; ++row) {                                                   \
        if (row >= sr0 && row < sr1) continue;                                              \
        T curr = dist[row + col * ldc];                                                     \
        int32_t p = parent[row + col * ldp];                                                \
        for (int i = 0; i < k; ++i) {                                                       \
          T prod = A[row + i * lda] + B[i + col * ldb];                                     \
          if (prod < curr) {                                                                \
            curr = prod;                                                                    \
            p = k_base + i;                                                                 \
          }                                                                                 \
        }                                                                                   \
        dist[row + col * ldc] = curr;                                                       \
        parent[row + col * ldp] = p;                                                        \
      }                                                                                     \
    }                                                                                       \
  }                                                                                         \
  static int NAME(int n, T *D, int64_t ld, int32_t *P, int64_t ldp, int b) {                \
    T *R = (T *)malloc(sizeof(T) * (size_t)b * (size_t)n);                                  \
    T *C = (T *)malloc(sizeof(T) * (size_t)b * (size_t)n);                                  \
    if (!R || !C) { free(R); free(C); return -2; }                                          \
    for (int k0 = 0; k0 < n; k0 += b) {                                                     \
      const int bb = n - k0 < b ? n - k0 : b;                                               \
      T *Dkk = D + k0 + k0 * ld;                                                            \
      int32_t *Pkk = P + k0 + k0 * ldp;                                                     \
      for (int k = 0; k < bb; ++k)                                                          \
        for (int j = 0; j < bb; ++j)                                                        \
          for (int i = 0; i < bb; ++i) {                                                    \
            T cand = Dkk[i + k * ld] + Dkk[k + j * ld];                                     \
            if (cand < Dkk[i + j * ld]) {                                                   \
              Dkk[i + j * ld] = cand;                                                       \
              Pkk[i + j * ldp] = k0 + k;                                                    \
            }                                                                               \
          }                                                                                 \
      for (int j = 0; j < n; ++j)                                                           \
        for (int i = 0; i < bb; ++i) R[i + (size_t)j * b] = D[(k0 + i) + j * ld];           \
      for (int j = 0; j < bb; ++j)                                                          \
        for (int i = 0; i < n; ++i) C[i + (size_t)j * n] = D[i + (k0 + j) * ld];            \
      NAME##_product(bb, n, bb, R + (size_t)k0 * b, b, R, b, D + k0, ld, P + k0, ldp, k0,   \
                     0, 0, k0, k0 + bb);                                                    \
      NAME##_product(n, bb, bb, C, n, C + k0, n, D + k0 * ld, ld, P + k0 * ldp, ldp, k0,    \
                     k0, k0 + bb, 0, 0);                                                    \
      NAME##_product(n, n, bb, D + k0 * ld, ld, D + k0, ld, D, ld, P, ldp, k0,              \
                     k0, k0 + bb, k0, k0 + bb);                                             \
    }                                                                                       \
    free(R);                                                                                \
    free(C);                                                                                \
    return 0;                                                                               \
  }

DEFINE_BLOCKED_FW(blocked_fw_f32, float)
DEFINE_BLOCKED_FW(blocked_fw_f64, double)

/* dtype: 0 = float, 1 = double.  dist (n x n, column-major, leading dimension ld)
 * and parent (int32, ldp) are updated in place; block is the diagonal block
 * size.  Returns 0, -1 for another element type, -2 when memory runs out. */
int oracle_apsp_blocked(int dtype, int n, void *dist, int64_t ld, int32_t *parent, int64_t ldp,
                        int block) {
  if (n <= 0 || block <= 0) return 0;
  if (dtype == 0) return blocked_fw_f32(n, (float *)dist, ld, parent, ldp, block);
  if (dtype == 1) return blocked_fw_f64(n, (double *)dist, ld, parent, ldp, block);
  return -1;
}
