/*
 * CPU oracle for semiring GEMM -- TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the GPU library is compared against.  It is
 * loaded by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
 * bench.py, and by nothing else: the shipped library (cuasr_amd/) never links,
 * imports or calls it.
 *
 * It restates, in plain C, the algorithm of the reference host SRGEMM
 *   tools/include/cuasr/reference/srgemm/host_srgemm.h:33-113
 * with the scalar operator semantics of
 *   include/cuasr/functional.h:46-49 (plus), :89-92 (multiplies),
 *   :132 (minimum), :172 (maximum), :212 (binary_and), :252 (binary_or)
 *   examples/01_userdefined_semiring/userdefined_semiring.cu:56-66 (binary_xor)
 * plus bitwise and/or, which the reference does not ship but which a
 * bit-packed GF(2) product needs.
 *
 * What is kept from the reference, because it decides the bits of the result:
 *   - the accumulator starts at the caller's add_identity          (:67-72)
 *   - k ascends and accum = add(mult(a, b), accum)                 (:75-91)
 *     (the product is the LEFT operand of add)
 *   - D = add(mult(alpha, accum), mult(beta, C)); C is always read (:94-109)
 *   - 32x32 output blocks, OpenMP over blocks (static, collapse 2) (:47-65);
 *     the upstream firstprivate clause names an undeclared variable, so
 *     upstream is serial; here the clause is simply dropped.
 * What is not kept, because it cannot change a result: bounds tests inside the
 * k loop (hoisted), the element accessor objects (plain strides here), and the
 * per-block A/B panels are packed so the compiler can vectorise over i.
 *
 * Parity status: every entry point below is pinned by tests/test_oracle.py
 * (the reference's 4x4x2 known-answer vector, a literal pure-Python triple
 * loop on ragged shapes and all layouts, float64 matmul / GF(2) bit-plane /
 * Floyd-Warshall closed forms).  None is "parity unpinned".
 *
 * The split-K model follows
 *   include/cuasr/gemm/kernel/srgemm_splitk_parallel.h:86-89, :136-142
 *     slice extent = ((K / tbk) / S) * tbk, last slice runs to K
 *   include/cuasr/reduction/kernel/reduce_split_k.h:162-227
 *     acc = identity; acc = add(acc, ws[s]) for s ascending;
 *     source = C if needed else identity; D = add(mult(alpha,acc), mult(beta,source))
 *   include/cuasr/gemm/epilogue/thread/semiring_linear_combination.h:118-125
 *     source needed  <=>  add_identity != mult(beta, mult_identity)
 *
 * The serial split-K model follows
 *   include/cuasr/gemm/kernel/srgemm.h:97-100, :184-189
 *     slice extent = ceil(ceil(K / tbk) / S) * tbk, slice z ends at min(K, (z+1) * extent)
 *   include/cuasr/gemm/kernel/srgemm.h:220-225, :249-320
 *     slices take turns on D in ascending order; slice 0's source is C, a later
 *     slice's source is D; a slice with no k range keeps acc = identity and still
 *     runs its epilogue
 *   include/cuasr/gemm/epilogue/thread/semiring_linear_combination.h:129-134, :152-183
 *     a later slice's beta is mult_identity; an unneeded source drops the add
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

enum { OP_PLUS = 0, OP_MULTIPLIES = 1, OP_MINIMUM = 2, OP_MAXIMUM = 3,
       OP_LOGICAL_AND = 4, OP_LOGICAL_OR = 5, OP_BIT_AND = 6, OP_BIT_OR = 7,
       OP_BIT_XOR = 8 };
enum { DT_F32 = 0, DT_F64 = 1, DT_I32 = 2, DT_U32 = 3, DT_F16 = 4, DT_I8 = 5 };
enum { LAYOUT_COLUMN_MAJOR = 0, LAYOUT_ROW_MAJOR = 1 };

#define BLK 32

/* scalar operators: (lhs, rhs) in the reference's argument order */
#define F_PLUS(l, r)        ((l) + (r))
#define F_MULTIPLIES(l, r)  ((l) * (r))
#define F_MINIMUM(l, r)     ((r) < (l) ? (r) : (l))
#define F_MAXIMUM(l, r)     ((l) < (r) ? (r) : (l))
#define F_LOGICAL_AND(l, r) ((l) && (r))
#define F_LOGICAL_OR(l, r)  ((l) || (r))
#define F_BIT_AND(l, r)     ((l) & (r))
#define F_BIT_OR(l, r)      ((l) | (r))
#define F_BIT_XOR(l, r)     ((l) ^ (r))
#define F_NE(l, r)          ((l) != (r))

/*
 * IEEE binary16, held as its bit pattern (gcc 11 on x86-64 has no _Float16).  The reference has no
 * half-precision kernels (README.md:11 names them as an aim); what its templates would compute with a
 * half type for every element (arch/srmma.h:65-92, functional.h:46-49, :89-92, :132, :172) is each
 * operator's exact result rounded once to binary16, ties to even.  Here: widen both operands to
 * binary32 (exact), operate in binary32, round to binary16.  That is the correctly rounded binary16
 * result: a product of two 11-bit significands is exact in 24 bits, and for a sum the binary32
 * rounding in between is harmless because 24 >= 2 * 11 + 2 (the classic double-rounding bound).
 * Comparisons are made on the widened values, so -0 == +0 and the operand returned is the reference's.
 */
typedef uint16_t h16;

static inline float h2f(h16 h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, bits;
  if (e == 0) {
    if (m == 0) {
      bits = sign;                                   /* zero */
    } else {                                         /* subnormal: value m * 2^-24 */
      int shift = 0;
      while (!(m & 0x400u)) { m <<= 1; ++shift; }
      bits = sign | ((uint32_t)(113 - shift) << 23) | ((m & 0x3ffu) << 13);
    }
  } else if (e == 31) {
    bits = sign | 0x7f800000u | (m << 13);           /* infinity, NaN */
  } else {
    bits = sign | ((e + 112) << 23) | (m << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static inline h16 f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (h16)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0)); /* inf / NaN */
  if (x >= 0x477ff000u) return (h16)(sign | 0x7c00u);   /* >= 65520 rounds to infinity */
  if (x < 0x33000001u) return (h16)sign;                /* <= 2^-25 rounds to zero (the tie goes to even = 0) */
  const int e = (int)(x >> 23) - 127;                   /* unbiased exponent, -25 .. 15 */
  uint32_t m = (x & 0x7fffffu) | 0x800000u;             /* 24-bit significand */
  int drop;                                             /* low bits of m that binary16 cannot hold */
  uint32_t base;
  if (e >= -14) { drop = 13; base = (uint32_t)(e + 15) << 10; m &= 0x7fffffu; }   /* normal */
  else { drop = 13 + (-14 - e); base = 0; }                                       /* subnormal: keep the leading 1 */
  const uint32_t kept = m >> drop, rest = m & ((1u << drop) - 1u), half = 1u << (drop - 1);
  uint32_t r = base + kept;                             /* a carry out of the significand bumps the exponent */
  if (rest > half || (rest == half && (kept & 1u))) ++r;
  return (h16)(sign | r);
}

/* entry points for the tests that pin the two conversions */
float oracle_half_to_float(uint16_t h) { return h2f(h); }
uint16_t oracle_float_to_half(float f) { return f2h(f); }

#define H_PLUS(l, r)        f2h(h2f(l) + h2f(r))
#define H_MULTIPLIES(l, r)  f2h(h2f(l) * h2f(r))
#define H_MINIMUM(l, r)     (h2f(r) < h2f(l) ? (r) : (l))
#define H_MAXIMUM(l, r)     (h2f(l) < h2f(r) ? (r) : (l))
#define H_LOGICAL_AND(l, r) ((h16)((h2f(l) != 0.0f && h2f(r) != 0.0f) ? 0x3c00u : 0u))
#define H_LOGICAL_OR(l, r)  ((h16)((h2f(l) != 0.0f || h2f(r) != 0.0f) ? 0x3c00u : 0u))
#define H_NE(l, r)          (h2f(l) != h2f(r))

#if defined(__x86_64__) && defined(__GNUC__) && !defined(ORACLE_NO_CLONES)
#define CLONES __attribute__((target_clones("avx512f", "avx2", "default")))
#else
#define CLONES
#endif

typedef struct {
  int m, n, k;
  const void *A; int64_t sa_m, sa_k;   /* element strides of A along m and k */
  const void *B; int64_t sb_k, sb_n;
  const void *C; int64_t sc_m, sc_n;
  void *D;       int64_t sd_m, sd_n;
  const void *alpha, *beta, *add_identity, *mult_identity;
  int k_begin, k_end;   /* accumulate range                                  */
  void *raw;            /* if non-NULL: write raw accumulators here, row-major
                           m x n, and skip the epilogue                     */
  const void *partials; /* if non-NULL: S row-major m x n slices to reduce   */
  int slices;
  int skip_source_if_unneeded; /* device-style epilogue (reduce kernel model) */
  int no_source_form;   /* with the above: an unneeded source drops the add,
                           D = mult(alpha, acc) (the SRGEMM kernel's epilogue) */
} job_t;

/*
 * One function per (type, add, mult).  acc[j][i]: i is the fast index so the
 * i loop vectorises; per element the order of operations is exactly
 * accum = add(mult(a, b), accum) for k ascending.
 */
#define DEFINE_KERNEL(NAME, T, TI, ADD, MUL, NE)                                  \
  CLONES static void NAME(const job_t *jb) {                                    \
    const int M = jb->m, N = jb->n;                                             \
    const TI *A = (const TI *)jb->A, *B = (const TI *)jb->B;                    \
    const T *C = (const T *)jb->C;                                              \
    T *D = (T *)jb->D;                                                          \
    const T alpha = *(const T *)jb->alpha, beta = *(const T *)jb->beta;         \
    const T ident = *(const T *)jb->add_identity;                               \
    const int k0 = jb->k_begin, k1 = jb->k_end, KK = k1 > k0 ? k1 - k0 : 0;     \
    const int mblocks = (M + BLK - 1) / BLK, nblocks = (N + BLK - 1) / BLK;     \
    _Pragma("omp parallel")                                                     \
    {                                                                           \
      T *Ap = (T *)malloc(sizeof(T) * BLK * (size_t)(KK > 0 ? KK : 1));         \
      T *Bp = (T *)malloc(sizeof(T) * BLK * (size_t)(KK > 0 ? KK : 1));         \
      _Pragma("omp for schedule(static) collapse(2)")                           \
      for (int rb = 0; rb < mblocks; ++rb) {                                    \
        for (int cb = 0; cb < nblocks; ++cb) {                                  \
          const int r0 = rb * BLK, c0 = cb * BLK;                               \
          const int mr = (M - r0) < BLK ? (M - r0) : BLK;                       \
          const int nc = (N - c0) < BLK ? (N - c0) : BLK;                       \
          T acc[BLK][BLK];                                                      \
          for (int j = 0; j < BLK; ++j)                                         \
            for (int i = 0; i < BLK; ++i) acc[j][i] = ident;                    \
          if (!jb->partials) {                                                  \
            for (int kk = 0; kk < KK; ++kk) {                                   \
              for (int i = 0; i < BLK; ++i)                                     \
                Ap[(size_t)kk * BLK + i] = i < mr                               \
                  ? (T)A[(int64_t)(r0 + i) * jb->sa_m + (int64_t)(k0 + kk) * jb->sa_k] \
                  : ident;                                                      \
              for (int j = 0; j < BLK; ++j)                                     \
                Bp[(size_t)kk * BLK + j] = j < nc                               \
                  ? (T)B[(int64_t)(k0 + kk) * jb->sb_k + (int64_t)(c0 + j) * jb->sb_n] \
                  : ident;                                                      \
            }                                                                   \
            for (int jq = 0; jq < BLK; jq += 4) {                               \
              for (int kk = 0; kk < KK; ++kk) {                                 \
                const T *ap = Ap + (size_t)kk * BLK;                            \
                const T *bp = Bp + (size_t)kk * BLK + jq;                       \
                for (int jj = 0; jj < 4; ++jj) {                                \
                  const T b = bp[jj];                                           \
                  for (int i = 0; i < BLK; ++i) {                               \
                    const T prod = MUL(ap[i], b);                               \
                    acc[jq + jj][i] = ADD(prod, acc[jq + jj][i]);               \
                  }                                                             \
                }                                                               \
              }                                                                 \
            }                                                                   \
          } else {                                                              \
            const T *ws = (const T *)jb->partials;                              \
            for (int s = 0; s < jb->slices; ++s)                                \
              for (int j = 0; j < nc; ++j)                                      \
                for (int i = 0; i < mr; ++i) {                                  \
                  const T w = ws[(size_t)s * M * N + (size_t)(r0 + i) * N + (c0 + j)]; \
                  acc[j][i] = ADD(acc[j][i], w);                                \
                }                                                               \
          }                                                                     \
          if (jb->raw) {                                                        \
            T *raw = (T *)jb->raw;                                              \
            for (int j = 0; j < nc; ++j)                                        \
              for (int i = 0; i < mr; ++i)                                      \
                raw[(size_t)(r0 + i) * N + (c0 + j)] = acc[j][i];               \
          } else {                                                              \
            int need = 1;                                                       \
            if (jb->skip_source_if_unneeded) {                                  \
              const T one = *(const T *)jb->mult_identity;                      \
              need = NE(ident, (T)MUL(beta, one));                              \
            }                                                                   \
            for (int j = 0; j < nc; ++j)                                        \
              for (int i = 0; i < mr; ++i) {                                    \
                const int64_t oc = (int64_t)(r0 + i) * jb->sc_m + (int64_t)(c0 + j) * jb->sc_n; \
                const int64_t od = (int64_t)(r0 + i) * jb->sd_m + (int64_t)(c0 + j) * jb->sd_n; \
                const T src = need ? C[oc] : ident;                             \
                const T lhs = MUL(alpha, acc[j][i]);                            \
                const T rhs = MUL(beta, src);                                   \
                if (!need && jb->no_source_form) D[od] = lhs;                   \
                else D[od] = ADD(lhs, rhs);                                     \
              }                                                                 \
          }                                                                     \
        }                                                                       \
      }                                                                         \
      free(Ap);                                                                 \
      free(Bp);                                                                 \
    }                                                                           \
  }

/* the literal triple loop, no blocking, no packing: an independent second
 * implementation used to cross-check the blocked one */
#define DEFINE_NAIVE(NAME, T, TI, ADD, MUL)                                     \
  static void NAME(const job_t *jb) {                                           \
    const TI *A = (const TI *)jb->A, *B = (const TI *)jb->B;                    \
    const T *C = (const T *)jb->C;                                              \
    T *D = (T *)jb->D;                                                          \
    const T alpha = *(const T *)jb->alpha, beta = *(const T *)jb->beta;         \
    const T ident = *(const T *)jb->add_identity;                               \
    for (int row = 0; row < jb->m; ++row)                                       \
      for (int col = 0; col < jb->n; ++col) {                                   \
        T accum = ident;                                                        \
        for (int kk = 0; kk < jb->k; ++kk) {                                    \
          const T a = (T)A[(int64_t)row * jb->sa_m + (int64_t)kk * jb->sa_k];   \
          const T b = (T)B[(int64_t)kk * jb->sb_k + (int64_t)col * jb->sb_n];   \
          const T prod = MUL(a, b);                                             \
          accum = ADD(prod, accum);                                             \
        }                                                                       \
        const T c = C[(int64_t)row * jb->sc_m + (int64_t)col * jb->sc_n];       \
        const T lhs = MUL(alpha, accum);                                        \
        const T rhs = MUL(beta, c);                                             \
        D[(int64_t)row * jb->sd_m + (int64_t)col * jb->sd_n] = ADD(lhs, rhs);   \
      }                                                                         \
  }

#define DEFINE_PAIR(T, TN, ADDN, MULN)                                          \
  DEFINE_KERNEL(blk_##TN##_##ADDN##_##MULN, T, T, F_##ADDN, F_##MULN, F_NE)     \
  DEFINE_NAIVE(nv_##TN##_##ADDN##_##MULN, T, T, F_##ADDN, F_##MULN)
#define DEFINE_HALF_PAIR(T, TN, ADDN, MULN)                                     \
  DEFINE_KERNEL(blk_##TN##_##ADDN##_##MULN, T, T, H_##ADDN, H_##MULN, H_NE)     \
  DEFINE_NAIVE(nv_##TN##_##ADDN##_##MULN, T, T, H_##ADDN, H_##MULN)
/* int8 operands, everything else int32: the element types of the reference's dp4a cores
 * (include/cuasr/gemm/threadblock/default_srmma_core_simt.h:747-757); a and b are widened first */
#define DEFINE_BYTE_PAIR(T, TN, ADDN, MULN)                                     \
  DEFINE_KERNEL(blk_##TN##_##ADDN##_##MULN, T, int8_t, F_##ADDN, F_##MULN, F_NE) \
  DEFINE_NAIVE(nv_##TN##_##ADDN##_##MULN, T, int8_t, F_##ADDN, F_##MULN)

/* add-ops x mult-ops available to floating types */
#define FOR_FLOAT_PAIRS(X, T, TN)                                               \
  X(T, TN, PLUS, PLUS) X(T, TN, PLUS, MULTIPLIES) X(T, TN, PLUS, MINIMUM)       \
  X(T, TN, PLUS, MAXIMUM) X(T, TN, PLUS, LOGICAL_AND)                           \
  X(T, TN, MINIMUM, PLUS) X(T, TN, MINIMUM, MULTIPLIES) X(T, TN, MINIMUM, MINIMUM) \
  X(T, TN, MINIMUM, MAXIMUM) X(T, TN, MINIMUM, LOGICAL_AND)                     \
  X(T, TN, MAXIMUM, PLUS) X(T, TN, MAXIMUM, MULTIPLIES) X(T, TN, MAXIMUM, MINIMUM) \
  X(T, TN, MAXIMUM, MAXIMUM) X(T, TN, MAXIMUM, LOGICAL_AND)                     \
  X(T, TN, LOGICAL_OR, PLUS) X(T, TN, LOGICAL_OR, MULTIPLIES)                   \
  X(T, TN, LOGICAL_OR, MINIMUM) X(T, TN, LOGICAL_OR, MAXIMUM)                   \
  X(T, TN, LOGICAL_OR, LOGICAL_AND)

/* the extra pairs integers get: anything with a bitwise operator in it */
#define FOR_INT_EXTRA_PAIRS(X, T, TN)                                           \
  X(T, TN, PLUS, BIT_AND) X(T, TN, MINIMUM, BIT_AND) X(T, TN, MAXIMUM, BIT_AND) \
  X(T, TN, LOGICAL_OR, BIT_AND)                                                 \
  X(T, TN, BIT_OR, PLUS) X(T, TN, BIT_OR, MULTIPLIES) X(T, TN, BIT_OR, MINIMUM) \
  X(T, TN, BIT_OR, MAXIMUM) X(T, TN, BIT_OR, LOGICAL_AND) X(T, TN, BIT_OR, BIT_AND) \
  X(T, TN, BIT_XOR, PLUS) X(T, TN, BIT_XOR, MULTIPLIES) X(T, TN, BIT_XOR, MINIMUM) \
  X(T, TN, BIT_XOR, MAXIMUM) X(T, TN, BIT_XOR, LOGICAL_AND) X(T, TN, BIT_XOR, BIT_AND)

FOR_FLOAT_PAIRS(DEFINE_PAIR, float, f32)
FOR_FLOAT_PAIRS(DEFINE_PAIR, double, f64)
FOR_FLOAT_PAIRS(DEFINE_PAIR, int32_t, i32)
FOR_INT_EXTRA_PAIRS(DEFINE_PAIR, int32_t, i32)
FOR_FLOAT_PAIRS(DEFINE_PAIR, uint32_t, u32)
FOR_INT_EXTRA_PAIRS(DEFINE_PAIR, uint32_t, u32)
FOR_FLOAT_PAIRS(DEFINE_HALF_PAIR, h16, f16)
FOR_FLOAT_PAIRS(DEFINE_BYTE_PAIR, int32_t, i8)
FOR_INT_EXTRA_PAIRS(DEFINE_BYTE_PAIR, int32_t, i8)

typedef void (*kernel_fn)(const job_t *);

#define LOOKUP_ROW(T, TN, ADDN, MULN)                                           \
  if (add_op == OP_##ADDN && mult_op == OP_##MULN)                              \
    return naive ? nv_##TN##_##ADDN##_##MULN : blk_##TN##_##ADDN##_##MULN;

static kernel_fn lookup(int dtype, int add_op, int mult_op, int naive) {
  switch (dtype) {
  case DT_F32: FOR_FLOAT_PAIRS(LOOKUP_ROW, float, f32) break;
  case DT_F64: FOR_FLOAT_PAIRS(LOOKUP_ROW, double, f64) break;
  case DT_I32:
    FOR_FLOAT_PAIRS(LOOKUP_ROW, int32_t, i32)
    FOR_INT_EXTRA_PAIRS(LOOKUP_ROW, int32_t, i32) break;
  case DT_U32:
    FOR_FLOAT_PAIRS(LOOKUP_ROW, uint32_t, u32)
    FOR_INT_EXTRA_PAIRS(LOOKUP_ROW, uint32_t, u32) break;
  case DT_F16: FOR_FLOAT_PAIRS(LOOKUP_ROW, h16, f16) break;
  case DT_I8:
    FOR_FLOAT_PAIRS(LOOKUP_ROW, int32_t, i8)
    FOR_INT_EXTRA_PAIRS(LOOKUP_ROW, int32_t, i8) break;
  default: break;
  }
  return 0;
}

static size_t dtype_size(int dtype) { return dtype == DT_F64 ? 8 : dtype == DT_F16 ? 2 : 4; }

static void set_strides(job_t *jb, int layout_a, int64_t lda, int layout_b,
                        int64_t ldb, int layout_c, int64_t ldc, int64_t ldd) {
  /* column-major: element (r, c) at r + c*ld; row-major: r*ld + c */
  jb->sa_m = layout_a == LAYOUT_COLUMN_MAJOR ? 1 : lda;
  jb->sa_k = layout_a == LAYOUT_COLUMN_MAJOR ? lda : 1;
  jb->sb_k = layout_b == LAYOUT_COLUMN_MAJOR ? 1 : ldb;
  jb->sb_n = layout_b == LAYOUT_COLUMN_MAJOR ? ldb : 1;
  jb->sc_m = layout_c == LAYOUT_COLUMN_MAJOR ? 1 : ldc;
  jb->sc_n = layout_c == LAYOUT_COLUMN_MAJOR ? ldc : 1;
  jb->sd_m = layout_c == LAYOUT_COLUMN_MAJOR ? 1 : ldd;
  jb->sd_n = layout_c == LAYOUT_COLUMN_MAJOR ? ldd : 1;
}

static void set_threads(int nthreads) {
#ifdef _OPENMP
  if (nthreads > 0) omp_set_num_threads(nthreads);
#else
  (void)nthreads;
#endif
}

int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* D = add(mult(alpha, A (x) B), mult(beta, C)); returns 0, or -1 when the
 * (dtype, add, mult) triple is not in the table.  naive != 0 selects the
 * literal triple loop (single thread). */
int oracle_srgemm(int dtype, int add_op, int mult_op, int m, int n, int k,
                  const void *alpha, const void *A, int64_t lda, int layout_a,
                  const void *B, int64_t ldb, int layout_b, const void *beta,
                  const void *C, int64_t ldc, void *D, int64_t ldd, int layout_c,
                  const void *add_identity, int nthreads, int naive) {
  kernel_fn fn = lookup(dtype, add_op, mult_op, naive);
  if (!fn) return -1;
  job_t jb;
  memset(&jb, 0, sizeof jb);
  jb.m = m; jb.n = n; jb.k = k;
  jb.A = A; jb.B = B; jb.C = C; jb.D = D;
  jb.alpha = alpha; jb.beta = beta; jb.add_identity = add_identity;
  jb.k_begin = 0; jb.k_end = k;
  set_strides(&jb, layout_a, lda, layout_b, ldb, layout_c, ldc, ldd);
  set_threads(nthreads);
  fn(&jb);
  return 0;
}

/* CPU model of the two-kernel parallel split-K: S partial products over the
 * reference's slice boundaries, then the reduction + epilogue.  tbk is the
 * tile depth the slice extent is rounded to (8 in every reference default). */
int oracle_srgemm_splitk(int dtype, int add_op, int mult_op, int m, int n, int k,
                         const void *alpha, const void *A, int64_t lda,
                         int layout_a, const void *B, int64_t ldb, int layout_b,
                         const void *beta, const void *C, int64_t ldc, void *D,
                         int64_t ldd, int layout_c, const void *add_identity,
                         const void *mult_identity, int slices, int tbk,
                         int nthreads) {
  kernel_fn fn = lookup(dtype, add_op, mult_op, 0);
  if (!fn || slices < 1 || tbk < 1) return -1;
  const size_t esz = dtype_size(dtype);
  void *ws = malloc(esz * (size_t)m * n * slices + 8);
  if (!ws) return -2;
  job_t jb;
  memset(&jb, 0, sizeof jb);
  jb.m = m; jb.n = n; jb.k = k;
  jb.A = A; jb.B = B; jb.C = C; jb.D = D;
  jb.alpha = alpha; jb.beta = beta; jb.add_identity = add_identity;
  jb.mult_identity = mult_identity;
  set_strides(&jb, layout_a, lda, layout_b, ldb, layout_c, ldc, ldd);
  set_threads(nthreads);
  const int ks = ((k / tbk) / slices) * tbk;
  for (int s = 0; s < slices; ++s) {
    jb.k_begin = s * ks;
    jb.k_end = (s + 1 == slices) ? k : (s + 1) * ks;
    jb.raw = (char *)ws + esz * (size_t)m * n * s;
    fn(&jb);
  }
  jb.raw = 0;
  jb.partials = ws;
  jb.slices = slices;
  jb.skip_source_if_unneeded = 1;
  fn(&jb);
  free(ws);
  return 0;
}

/* CPU model of the serial split-K: the slices' epilogues applied to D one after
 * the other, slice 0 first.  tbk is the tile depth the slice extent is rounded
 * to (8 in every reference default). */
int oracle_srgemm_splitk_serial(int dtype, int add_op, int mult_op, int m, int n,
                                int k, const void *alpha, const void *A,
                                int64_t lda, int layout_a, const void *B,
                                int64_t ldb, int layout_b, const void *beta,
                                const void *C, int64_t ldc, void *D, int64_t ldd,
                                int layout_c, const void *add_identity,
                                const void *mult_identity, int slices, int tbk,
                                int nthreads) {
  kernel_fn fn = lookup(dtype, add_op, mult_op, 0);
  if (!fn || slices < 1 || tbk < 1) return -1;
  job_t jb;
  memset(&jb, 0, sizeof jb);
  jb.m = m; jb.n = n; jb.k = k;
  jb.A = A; jb.B = B; jb.D = D;
  jb.alpha = alpha; jb.add_identity = add_identity;
  jb.mult_identity = mult_identity;
  jb.skip_source_if_unneeded = 1;
  jb.no_source_form = 1;
  set_threads(nthreads);
  const int64_t iters = ((int64_t)k + tbk - 1) / tbk;
  const int64_t ks = ((iters + slices - 1) / slices) * tbk;
  for (int z = 0; z < slices; ++z) {
    const int64_t b = z * ks, e = (z + 1) * ks;
    jb.k_begin = (int)(b < k ? b : k);
    jb.k_end = (int)(e < k ? e : k);
    if (z == 0) {
      jb.C = C; jb.beta = beta;
      set_strides(&jb, layout_a, lda, layout_b, ldb, layout_c, ldc, ldd);
    } else {
      jb.C = D; jb.beta = mult_identity;
      set_strides(&jb, layout_a, lda, layout_b, ldb, layout_c, ldd, ldd);
    }
    fn(&jb);
  }
  return 0;
}
