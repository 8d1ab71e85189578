/*
 * CPU oracle for the min-plus product with predecessor tracking -- TEST
 * INFRASTRUCTURE ONLY (see host_srgemm.c: only tests/, smoke() and the
 * cpu_baseline leg of bench.py may use this library).
 *
 * Restates cpu_fwgemm_naive,
 *   test/regress/include/fwgpu/cpu_srgemm.hpp:20-48
 * for column-major A (m x k), B (k x n), dist and parent (m x n):
 *   for every (row, col): curr = dist, p = parent; for k ascending:
 *   prod = A[row,k] + B[k,col]; if (prod < curr) { curr = prod; p = k; }
 *   then dist = curr, parent = p.                                   (:35-45)
 * The upstream body runs all three loops to n (its k parameter is shadowed,
 * :32-38), which is the signature's meaning only on square operands; here the
 * loops run to m, n and k as the signature says, which is the same thing on the
 * square matrices of an all-pairs shortest-path step.  Upstream indexes parent
 * with ldc; here it has a leading dimension of its own.
 *
 * Parity status: pinned by tests/test_oracle.py -- dist against the min-plus
 * SRGEMM oracle (itself pinned), parent against numpy's first-occurrence argmin
 * and the strict-improvement rule, a hand-worked graph, and paths rebuilt from
 * parent after repeated squaring against scipy's Floyd-Warshall.
 */
#include <stdint.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define DEFINE_FWGEMM(NAME, T)                                                      \
  static void NAME(int m, int n, int k, const T *A, int64_t lda, const T *B,        \
                   int64_t ldb, T *dist, int64_t ldc, int32_t *parent, int64_t ldp) { \
    _Pragma("omp parallel for schedule(static)")                                    \
    for (int col = 0; col < n; ++col) {                                             \
      for (int row = 0; row < m; ++row) {                                           \
        T curr = dist[row + col * ldc];                                             \
        int32_t p = parent[row + col * ldp];                                        \
        for (int i = 0; i < k; ++i) {                                               \
          T prod = A[row + i * lda] + B[i + col * ldb];                             \
          if (prod < curr) {                                                        \
            curr = prod;                                                            \
            p = i;                                                                  \
          }                                                                         \
        }                                                                           \
        dist[row + col * ldc] = curr;                                               \
        parent[row + col * ldp] = p;                                                \
      }                                                                             \
    }                                                                               \
  }

DEFINE_FWGEMM(fwgemm_f32, float)
DEFINE_FWGEMM(fwgemm_f64, double)

/* dtype: 0 = float, 1 = double (the SRGEMM oracle's numbering).  Returns 0, or
 * -1 for another element type. */
int oracle_fwgemm(int dtype, int m, int n, int k, const void *A, int64_t lda,
                  const void *B, int64_t ldb, void *dist, int64_t ldc,
                  int32_t *parent, int64_t ldp, int nthreads) {
#ifdef _OPENMP
  if (nthreads > 0) omp_set_num_threads(nthreads);
#else
  (void)nthreads;
#endif
  if (dtype == 0)
    fwgemm_f32(m, n, k, (const float *)A, lda, (const float *)B, ldb, (float *)dist, ldc, parent, ldp);
  else if (dtype == 1)
    fwgemm_f64(m, n, k, (const double *)A, lda, (const double *)B, ldb, (double *)dist, ldc, parent, ldp);
  else
    return -1;
  return 0;
}
