/*
 * cuasr_amd C ABI: semiring GEMM (SRGEMM) on AMD Instinct MI355X (gfx950).
 *
 *     D = add( mult(alpha, A (x) B), mult(beta, C) )
 *     (A (x) B)[i][j] = add over k of mult(A[i][k], B[k][j]), starting from add_identity
 *
 * This is the boundary the C++ operator templates in include/cuasr/ call, and
 * the one a foreign-function binding would bind.  Plain C types only; all
 * matrix pointers are device pointers owned by the caller; nothing here
 * allocates, frees or synchronises.  Every call is asynchronous on `stream`
 * (a hipStream_t passed as void*, NULL = the default stream).
 *
 * Reference interfaces replaced (paths relative to the cuASR tree):
 *   cuasr_amd_srgemm                  device::Srgemm::operator()/run
 *                                     include/cuasr/gemm/device/srgemm.h:303-356
 *   cuasr_amd_srgemm_can_implement    device::Srgemm::can_implement  :196-215
 *                                     kernel::Srgemm::can_implement
 *                                     include/cuasr/gemm/kernel/srgemm.h:118-153
 *   cuasr_amd_splitk_workspace_bytes  device::SrgemmSplitKParallel::get_workspace_size
 *                                     include/cuasr/gemm/device/srgemm_splitk_parallel.h:226-235
 *   cuasr_amd_srgemm_splitk           device::SrgemmSplitKParallel::initialize/run
 *                                     include/cuasr/gemm/device/srgemm_splitk_parallel.h:238-357
 *   cuasr_amd_srgemm_splitk_serial    device::Srgemm<..., SplitKSerial = true>
 *                                     include/cuasr/gemm/device/srgemm.h:218-282
 *   status codes                      cutlass::Status as used by the reference
 *                                     test/device/testbed.h:24-46
 */
#ifndef CUASR_AMD_H
#define CUASR_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CUASR_AMD_ABI_VERSION 1

/* Same names and order as cutlass::Status, so static_cast<int>(status) agrees. */
typedef enum cuasr_amd_status {
  CUASR_AMD_SUCCESS = 0,
  CUASR_AMD_ERROR_MISALIGNED_OPERAND = 1,
  CUASR_AMD_ERROR_INVALID_DATA_TYPE = 2,
  CUASR_AMD_ERROR_INVALID_LAYOUT = 3,
  CUASR_AMD_ERROR_INVALID_PROBLEM = 4,
  CUASR_AMD_ERROR_NOT_SUPPORTED = 5,
  CUASR_AMD_ERROR_WORKSPACE_NULL = 6,
  CUASR_AMD_ERROR_INTERNAL = 7,
  CUASR_AMD_ERROR_ARCH_MISMATCH = 8,
  CUASR_AMD_ERROR_INSUFFICIENT_DRIVER = 9,
  CUASR_AMD_ERROR_MEMORY_ALLOCATION = 10,
  CUASR_AMD_INVALID = 11
} cuasr_amd_status;

/* Scalar operators.  (lhs, rhs) semantics follow include/cuasr/functional.h:
 * minimum = rhs < lhs ? rhs : lhs, maximum = lhs < rhs ? rhs : lhs,
 * logical_and/or produce 0 or 1 (functional.h:212, :252); bit_* are bitwise
 * and only defined for the integer element types. */
typedef enum cuasr_amd_op {
  CUASR_AMD_OP_PLUS = 0,
  CUASR_AMD_OP_MULTIPLIES = 1,
  CUASR_AMD_OP_MINIMUM = 2,
  CUASR_AMD_OP_MAXIMUM = 3,
  CUASR_AMD_OP_LOGICAL_AND = 4,
  CUASR_AMD_OP_LOGICAL_OR = 5,
  CUASR_AMD_OP_BIT_AND = 6,
  CUASR_AMD_OP_BIT_OR = 7,
  CUASR_AMD_OP_BIT_XOR = 8
} cuasr_amd_op;

typedef enum cuasr_amd_dtype {
  CUASR_AMD_F32 = 0,
  CUASR_AMD_F64 = 1,
  CUASR_AMD_I32 = 2,
  CUASR_AMD_U32 = 3,
  /* IEEE binary16 in A, B, C, D, the scalars and the accumulator: every operator rounds its result to
   * binary16, as the reference's templates do when they are instantiated with cutlass::half_t for all
   * element types (the reference names half precision as an aim only, README.md:11) */
  CUASR_AMD_F16 = 4,
  /* A and B hold int8; C, D, the scalars and the accumulator are int32 -- the element types of the reference's
   * dp4a cores (include/cuasr/gemm/threadblock/default_srmma_core_simt.h:747-757: ElementA = ElementB = int8_t,
   * ElementC a parameter; they are never instantiated there).  Every operator acts on the values widened to
   * int32; lda / ldb count int8 elements, ldc / ldd int32 elements */
  CUASR_AMD_I8 = 5
} cuasr_amd_dtype;

typedef enum cuasr_amd_layout {
  CUASR_AMD_COLUMN_MAJOR = 0, /* element (r, c) at r + c * ld */
  CUASR_AMD_ROW_MAJOR = 1     /* element (r, c) at r * ld + c */
} cuasr_amd_layout;

/* Which kernel family runs.  AUTO picks the fastest one that is valid for the
 * problem; the others exist so tests can pin every family against the oracle. */
typedef enum cuasr_amd_kernel {
  CUASR_AMD_KERNEL_AUTO = 0,
  CUASR_AMD_KERNEL_NAIVE = 1, /* one thread per output element               */
  CUASR_AMD_KERNEL_VALU = 2,  /* LDS-staged, register-blocked vector-ALU tile */
  CUASR_AMD_KERNEL_MFMA = 3,  /* matrix-core assisted tile.  For CUASR_AMD_F16 plus-times this family accumulates
                                 in float and rounds D to binary16 once (the reference's ElementAccumulator =
                                 float); AUTO never picks it there, because AUTO's binary16 sums are rounded
                                 term by term like the reference's all-half instantiation */
  CUASR_AMD_KERNEL_VALU_DIRECT = 4, /* vector-ALU tile fed by direct-to-LDS loads;
                                       needs 16-byte aligned, vector-sized operands */
  CUASR_AMD_KERNEL_VALU_STREAMK = 5 /* the same tile with the k-tiles of all output tiles shared out evenly over
                                       two workgroups per compute unit, for outputs whose tiles do not fill
                                       whole rounds of the chip; 4-byte min/max-plus, max-min, min-max, xor-and,
                                       or-and with alpha = the multiplicative identity given by value; not for
                                       split-K or batches.  Two launches: D <- the source term, then the product
                                       folded into D (D may alias C as always) */
} cuasr_amd_kernel;

/* One element of the problem's type; read through the member `dtype` names. */
typedef union cuasr_amd_scalar {
  float f32;
  double f64;
  int32_t i32;
  uint32_t u32;
  uint16_t f16;  /* the bit pattern of an IEEE binary16 value (C has no portable type for it) */
  uint64_t bits;
} cuasr_amd_scalar;

/*
 * Problem descriptor (device::Srgemm::Arguments, device/srgemm.h:139-183, plus
 * what the reference fixes at compile time through its template parameters).
 * A is m x k, B is k x n, C and D are m x n and share layout_c.  ld* are in
 * elements.  D may alias C.  C is not dereferenced when the source is not
 * needed, i.e. when add_identity == mult(beta, mult_identity)
 * (epilogue/thread/semiring_linear_combination.h:118-125).
 * alpha_ptr / beta_ptr, when non-NULL, are device pointers to one element
 * that override alpha / beta (same file, :88-99, :112-115).
 */
typedef struct cuasr_amd_srgemm_desc {
  int32_t add_op;          /* cuasr_amd_op */
  int32_t mult_op;         /* cuasr_amd_op */
  int32_t dtype;           /* cuasr_amd_dtype: A, B, C, D and accumulator (CUASR_AMD_I8: int8 A and B, int32 the rest) */
  int32_t layout_a;        /* cuasr_amd_layout */
  int32_t layout_b;
  int32_t layout_c;
  int32_t m, n, k;
  int32_t split_k_slices;  /* 1 for cuasr_amd_srgemm; >= 1 for the split-K call */
  const void *A; int64_t lda;
  const void *B; int64_t ldb;
  const void *C; int64_t ldc;
  void *D;       int64_t ldd;
  cuasr_amd_scalar alpha;
  cuasr_amd_scalar beta;
  cuasr_amd_scalar add_identity;   /* AdditionOp::Identity        */
  cuasr_amd_scalar mult_identity;  /* MultiplicationOp::Identity  */
  const void *alpha_ptr;
  const void *beta_ptr;
  int32_t kernel;          /* cuasr_amd_kernel */
  int32_t reserved;        /* must be 0 */
} cuasr_amd_srgemm_desc;

/* ABI version the library was built with. */
int cuasr_amd_abi_version(void);

/* Static text for a status code. */
const char *cuasr_amd_status_string(int status);

/* Validate a descriptor without touching the device.  Returns
 * CUASR_AMD_ERROR_INVALID_PROBLEM for negative extents, ld smaller than the
 * extent, or split_k_slices != 1; CUASR_AMD_ERROR_MISALIGNED_OPERAND for
 * pointers not aligned to the element size; CUASR_AMD_ERROR_INVALID_DATA_TYPE /
 * _INVALID_LAYOUT for unknown enums; CUASR_AMD_ERROR_NOT_SUPPORTED for an
 * operator pair the element type does not define (bitwise on floating point)
 * or a kernel family that cannot run the problem. */
int cuasr_amd_srgemm_can_implement(const cuasr_amd_srgemm_desc *desc);

/* Launch one SRGEMM.  Fails with CUASR_AMD_ERROR_INVALID_PROBLEM when
 * split_k_slices > 1 (device/srgemm.h:198-200). */
int cuasr_amd_srgemm(const cuasr_amd_srgemm_desc *desc, void *stream);

/* A batch of SRGEMMs that share one descriptor: product i works on the
 * descriptor's A, B, C, D advanced by i * stride_a, i * stride_b, i * stride_c,
 * i * stride_d ELEMENTS (the reference only names batched operation as an aim,
 * README.md:11, and has no such call).  Stride 0 shares an operand between all
 * products; the outputs must lie at least one matrix apart, strides must not be
 * negative (CUASR_AMD_ERROR_INVALID_PROBLEM otherwise).  The kernel family is
 * chosen once, for the whole batch (what fills the chip is the batch, not one
 * product); on the vector-ALU tiles, and on the matrix-core tiles for products
 * whose k is a multiple of 16 and whose operands (batch strides included) are
 * 16-byte aligned, the product index is part of the grid, so a batch of many
 * small products is a single launch; the other matrix-core kernels and the
 * naive kernel run the products one after the other on the stream.  Each
 * product's result is that of a single cuasr_amd_srgemm on its operands. */
int cuasr_amd_srgemm_batched(const cuasr_amd_srgemm_desc *desc, int batch, int64_t stride_a,
                             int64_t stride_b, int64_t stride_c, int64_t stride_d, void *stream);

/* Bytes of device workspace the split-K call needs:
 * sizeof(element of C) * m * n * split_k_slices. */
size_t cuasr_amd_splitk_workspace_bytes(const cuasr_amd_srgemm_desc *desc);

/* Two launches on `stream`: partial products of `split_k_slices` K-slices into
 * `workspace`, then a reduction with the semiring's add and the epilogue.
 * CUASR_AMD_ERROR_WORKSPACE_NULL when workspace is NULL
 * (device/srgemm_splitk_parallel.h:247-249).  The workspace must be aligned to
 * the element size; a workspace that is not 16-byte aligned keeps AUTO off the
 * direct-to-LDS tiles (they store 16-byte vectors), and a forced
 * CUASR_AMD_KERNEL_VALU_DIRECT is then refused with
 * CUASR_AMD_ERROR_MISALIGNED_OPERAND. */
int cuasr_amd_srgemm_splitk(const cuasr_amd_srgemm_desc *desc, void *workspace,
                            void *stream);

/* The second kernel of the parallel split-K on its own (reduction::kernel::ReduceSplitK,
 * include/cuasr/reduction/kernel/reduce_split_k.h:56-238, which the reference launches
 * at device/srgemm_splitk_parallel.h:348): folds the `split_k_slices` partial tiles
 * that a slice kernel left in `workspace` (slice z at workspace + z * m * n elements,
 * row-major in the orientation the slice kernel wrote them) with the semiring's add,
 * slice 0 first, and applies the epilogue D = add(mult(alpha, acc), mult(beta, C)).
 * For callers that produce or keep the partial tiles themselves, and for timing the
 * reduction alone.  Arguments and errors as cuasr_amd_srgemm_splitk. */
int cuasr_amd_reduce_splitk(const cuasr_amd_srgemm_desc *desc, void *workspace, void *stream);

/* Split-K for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart
 * in the reference, whose split-K always takes the caller's workspace
 * (device/srgemm_splitk_parallel.h:238-249).  Same result as
 * cuasr_amd_srgemm_splitk, bit for bit; the partial tiles go to a fixed array of
 * CUASR_AMD_STATIC_WORKSPACE_BYTES inside the library's device image (one copy
 * per GPU, held until the process ends) instead of a caller workspace.  The call
 * makes no hipMalloc / hipFree and no allocating library call; its first use on
 * a device looks the array's address up once (make that first call outside a
 * graph capture).  CUASR_AMD_ERROR_MEMORY_ALLOCATION when
 * sizeof(element) * m * n * split_k_slices exceeds the array.  All calls on one
 * GPU share the array: calls that may overlap in time on one GPU (different
 * streams, several host threads) race on it and must be ordered by the caller;
 * calls on one stream are ordered by the stream. */
#define CUASR_AMD_STATIC_WORKSPACE_BYTES (16u << 20)
int cuasr_amd_srgemm_splitk_static(const cuasr_amd_srgemm_desc *desc, void *stream);

/* Serial split-K (device::Srgemm with SplitKSerial = true,
 * include/cuasr/gemm/device/srgemm.h:218-282; include/cuasr/gemm/kernel/srgemm.h:249-320).
 * The result is the reference's chain of epilogues, slice 0 first:
 *   D_0 = add(mult(alpha, acc_0), mult(beta, C))     (mult(alpha, acc_0) if C is not needed)
 *   D_z = add(mult(alpha, acc_z), mult(mult_identity, D_{z-1}))   for z = 1 .. slices-1
 * The reference orders the slices' workgroups with one semaphore per output tile
 * and reduces in place in D, so its workspace is one int per tile.  Here the
 * slices run unordered into the workspace and one reduction kernel replays the
 * chain, so the workspace holds the partial products: callers must size it with
 * cuasr_amd_splitk_serial_workspace_bytes, which returns
 * sizeof(element) * m * n * split_k_slices, or 0 when split_k_slices == 1
 * (then the call is cuasr_amd_srgemm and the workspace may be NULL).
 * CUASR_AMD_ERROR_WORKSPACE_NULL when split_k_slices > 1 and workspace is NULL
 * (device/srgemm.h:248-251). */
size_t cuasr_amd_splitk_serial_workspace_bytes(const cuasr_amd_srgemm_desc *desc);
int cuasr_amd_srgemm_splitk_serial(const cuasr_amd_srgemm_desc *desc, void *workspace,
                                   void *stream);

/* Min-plus product with predecessor tracking, the step of an all-pairs
 * shortest-path computation that can rebuild its paths
 * (cpu_fwgemm_naive, test/regress/include/fwgpu/cpu_srgemm.hpp:20-48; the
 * reference has this on the CPU only).  A (m x k), B (k x n), dist and parent
 * (m x n) are column-major device matrices with leading dimensions in elements;
 * dtype is CUASR_AMD_F32 or CUASR_AMD_F64, parent holds int32.  In place, for
 * every (row, col):
 *   scan k ascending; prod = A[row,k] + B[k,col];
 *   if (prod < dist[row,col]) { dist[row,col] = prod; parent[row,col] = k; }
 * Elements that do not improve keep both values.  Results are bit-identical to
 * that scan for operands free of NaN and -infinity (+infinity = no edge).
 * A and B must not overlap dist.  kernel: CUASR_AMD_KERNEL_AUTO, _NAIVE (one
 * thread per element) or _VALU (LDS-staged tile).  Errors as for cuasr_amd_srgemm. */
int cuasr_amd_fwgemm(int dtype, int m, int n, int k, const void *A, int64_t lda,
                     const void *B, int64_t ldb, void *dist, int64_t ldc,
                     int32_t *parent, int64_t ldp, int kernel, void *stream);

/* All-pairs shortest paths by repeated squaring on an n x n distance matrix
 * (the application README.md:338-342 of the reference motivates): `iterations`
 * times, dist is copied into the workspace and cuasr_amd_fwgemm(workspace,
 * workspace, dist, parent) is run; iterations = 0 means ceil(log2(n - 1)), which
 * covers every path.  parent[i,j] = k says the shortest i -> j path found is the
 * i -> k path followed by the k -> j path; an entry the caller initialised (say
 * to -1) and that never changed means the direct edge.  The workspace holds
 * cuasr_amd_apsp_workspace_bytes(dtype, n) = 2 * sizeof(element) * n * n bytes
 * (the snapshot and its transpose, in which the search for the first minimising
 * k reads contiguous memory); CUASR_AMD_ERROR_WORKSPACE_NULL without it.  Asynchronous on the stream, no
 * allocation, no host synchronisation. */
size_t cuasr_amd_apsp_workspace_bytes(int dtype, int n);
int cuasr_amd_apsp_squaring(int dtype, int n, void *dist, int64_t ld, int32_t *parent,
                            int64_t ldp, void *workspace, int iterations, void *stream);

/* All-pairs shortest paths by blocked Floyd-Warshall with predecessor tracking:
 * n^3 products instead of the n^3 * log2(n) of repeated squaring.  The reference
 * has no such routine; it is built from the reference's block, the product of
 * cpu_fwgemm_naive (test/regress/include/fwgpu/cpu_srgemm.hpp:20-48), for the
 * application its README names (README.md:338-342).  For every diagonal block of
 * 128 vertices: Floyd-Warshall inside the block; block row and block column
 * through the closed block; every other element through block column x block
 * row.  dist (n x n, column-major, leading dimension ld) and parent (int32, ldp)
 * are updated in place: on return dist holds the shortest distances and
 * parent[i,j] = k says the path found is the i -> k path followed by the k -> j
 * path (an entry the caller initialised, say to -1, that never changed: the
 * direct edge).  Weights must be free of NaN and -infinity, +infinity = no
 * edge, no negative cycles.  Sums along a path are formed in the blocked order,
 * so on weights whose sums round, distances can differ in the last bits from
 * those of cuasr_amd_apsp_squaring (both are sums of the same edges).  The
 * workspace holds cuasr_amd_apsp_blocked_workspace_bytes(dtype, n) bytes
 * (3 * 128 * (n + 128) elements, n rounded up to a multiple of 4) and is 16-byte
 * aligned; CUASR_AMD_ERROR_WORKSPACE_NULL without it.  Asynchronous on the
 * stream, no allocation, no host synchronisation. */
size_t cuasr_amd_apsp_blocked_workspace_bytes(int dtype, int n);
int cuasr_amd_apsp_blocked(int dtype, int n, void *dist, int64_t ld, int32_t *parent,
                           int64_t ldp, void *workspace, void *stream);

/* The same with the choice of how a block step updates its block row and block column made by the
 * caller: CUASR_AMD_PANELS_AUTO (what cuasr_amd_apsp_blocked does: PAIRED below n = 16257, TILED from
 * there on, where each panel product fills the chip on its own), CUASR_AMD_PANELS_PAIRED (both products
 * in one launch of the one-thread-per-element kernel) or CUASR_AMD_PANELS_TILED (two launches of the
 * tiled kernel and a transposing copy of the updated block column).  Results do not depend on it.
 * CUASR_AMD_ERROR_INVALID_PROBLEM for any other value. */
#define CUASR_AMD_PANELS_AUTO 0
#define CUASR_AMD_PANELS_PAIRED 1
#define CUASR_AMD_PANELS_TILED 2
int cuasr_amd_apsp_blocked_panels(int dtype, int n, void *dist, int64_t ld, int32_t *parent,
                                  int64_t ldp, void *workspace, int panels, void *stream);

/* Name of the kernel family AUTO would choose for this descriptor
 * ("naive", "valu", "valu_direct", "valu_streamk", "mfma"; "valu_direct+valu" when a block of the output runs on
 * the direct-to-LDS tile and the strips around it on the staged one), or NULL if the descriptor
 * is invalid. */
const char *cuasr_amd_selected_kernel(const cuasr_amd_srgemm_desc *desc);

/* The same for cuasr_amd_srgemm_batched with these strides: the family, followed by ", a launch per product"
 * when the product index does not go into the grid ("a launch per product" alone: every product chooses as
 * cuasr_amd_selected_kernel says).  A batch whose strides are not multiples of 16 bytes stays off the
 * direct-to-LDS tiles, whose vector loads need that alignment for every product, and runs on the staged tile.
 * NULL for an invalid call. */
const char *cuasr_amd_selected_kernel_batched(const cuasr_amd_srgemm_desc *desc, int batch, int64_t stride_a,
                                              int64_t stride_b, int64_t stride_c, int64_t stride_d);

#ifdef __cplusplus
}
#endif
#endif /* CUASR_AMD_H */
