// C ABI of libcuasr_amd: validation, transposition of column-major outputs,
// kernel-family selection and launch.  Host-side counterpart of
// include/cuasr/gemm/device/srgemm.h:196-356 and
// include/cuasr/gemm/device/srgemm_splitk_parallel.h:220-357.
#include <atomic>

#include "semiring.h"

namespace cuasr_amd {

launch_fn find_valu_f32(int, int);
launch_fn find_valu_f64(int, int);
launch_fn find_valu_i32(int, int);
launch_fn find_valu_u32(int, int);
launch_fn find_valu_f16(int, int);
launch_fn find_valu_i8(int, int);
launch_fn find_mfma_f32(int, int);
launch_fn find_mfma_f64(int, int);
launch_fn find_mfma_i8(int, int);
launch_fn find_mfma_f16(int, int);
launch_fn find_direct_f32(int, int);
launch_fn find_direct_i32(int, int);
launch_fn find_direct_u32(int, int);
launch_fn find_direct_f64(int, int);
streamk_fn find_streamk_f32(int, int);
streamk_fn find_streamk_i32(int, int);
streamk_fn find_streamk_u32(int, int);
bool direct_can_run(const Problem &);
bool direct64_can_run(const Problem &);
bool mfma_f32_can_run(const Problem &);
bool mfma_f64_can_run(const Problem &);
bool mfma_direct_f32_can_run(const Problem &);
bool mfma_direct_f64_can_run(const Problem &);

launch_fn find_or_and_on_masks(int dtype);

launch_fn find_valu(int dtype, int add_op, int mult_op) {
  if (add_op == kLogicalOr && mult_op == kLogicalAnd)
    if (launch_fn f = find_or_and_on_masks(dtype)) return f;  // float, double: the packed mask tile for large outputs
  switch (dtype) {
    case CUASR_AMD_F32: return find_valu_f32(add_op, mult_op);
    case CUASR_AMD_F64: return find_valu_f64(add_op, mult_op);
    case CUASR_AMD_I32: return find_valu_i32(add_op, mult_op);
    case CUASR_AMD_U32: return find_valu_u32(add_op, mult_op);
    case CUASR_AMD_F16: return find_valu_f16(add_op, mult_op);
    case CUASR_AMD_I8: return find_valu_i8(add_op, mult_op);
    default: return nullptr;
  }
}

launch_fn find_direct(int dtype, int add_op, int mult_op) {
  switch (dtype) {
    case CUASR_AMD_F32: return find_direct_f32(add_op, mult_op);
    case CUASR_AMD_I32: return find_direct_i32(add_op, mult_op);
    case CUASR_AMD_U32: return find_direct_u32(add_op, mult_op);
    case CUASR_AMD_F64: return find_direct_f64(add_op, mult_op);
    default: return nullptr;
  }
}

streamk_fn find_streamk(int dtype, int add_op, int mult_op) {
  switch (dtype) {
    case CUASR_AMD_F32: return find_streamk_f32(add_op, mult_op);
    case CUASR_AMD_I32: return find_streamk_i32(add_op, mult_op);
    case CUASR_AMD_U32: return find_streamk_u32(add_op, mult_op);
    default: return nullptr;
  }
}

launch_fn find_mfma(int dtype, int add_op, int mult_op) {
  if (dtype == CUASR_AMD_F32) return find_mfma_f32(add_op, mult_op);
  if (dtype == CUASR_AMD_F64) return find_mfma_f64(add_op, mult_op);
  if (dtype == CUASR_AMD_I8) return find_mfma_i8(add_op, mult_op);
  if (dtype == CUASR_AMD_F16) return find_mfma_f16(add_op, mult_op);  // (float accumulation: by request only)
  return nullptr;
}

// bytes per element of C, D, the scalars and the workspace; and of A and B (int8 operands meet int32 everything else)
static size_t elem_size(int dtype) { return dtype == CUASR_AMD_F64 ? 8 : dtype == CUASR_AMD_F16 ? 2 : 4; }
static size_t operand_size(int dtype) { return dtype == CUASR_AMD_I8 ? 1 : elem_size(dtype); }

static bool is_bitwise(int op) { return op == kBitAnd || op == kBitOr || op == kBitXor; }

// add must be associative and commutative with an identity; mult is any of the
// "times-like" operators.  Both lists mirror what the reference can spell.
static bool valid_add(int op) {
  return op == kPlus || op == kMinimum || op == kMaximum || op == kLogicalOr || op == kBitOr || op == kBitXor ||
         op == kMultiplies || op == kLogicalAnd || op == kBitAnd;
}
static bool valid_mult(int op) { return op >= kPlus && op <= kBitXor; }

static Problem canonical(const cuasr_amd_srgemm_desc *d);

// the matrix-core tiles use 16-byte loads and so need aligned, vector-sized operands
static bool mfma_usable(const cuasr_amd_srgemm_desc *d) {
  if (!find_mfma(d->dtype, d->add_op, d->mult_op)) return false;
  if (d->dtype == CUASR_AMD_I8) return true;  // its kernel has a guarded form for every extent and alignment
  if (d->dtype == CUASR_AMD_F16) return d->split_k_slices == 1;  // likewise; its float sums have no binary16 split-K form
  return d->dtype == CUASR_AMD_F64 ? mfma_f64_can_run(canonical(d)) : mfma_f32_can_run(canonical(d));
}

// the direct-to-LDS tiles need aligned, vector-sized operands as well
static bool direct_usable(const cuasr_amd_srgemm_desc *d) {
  if (!find_direct(d->dtype, d->add_op, d->mult_op)) return false;
  return d->dtype == CUASR_AMD_F64 ? direct64_can_run(canonical(d)) : direct_can_run(canonical(d));
}

// The stream-K form of the direct tile: exact only for an add that does not depend on the order or grouping of
// its terms, with alpha = the multiplicative identity given by value, on the panel forms that have a hand-scheduled loop.
static bool streamk_usable(const cuasr_amd_srgemm_desc *d) {
  if (!find_streamk(d->dtype, d->add_op, d->mult_op) || !direct_usable(d)) return false;
  const Problem c = canonical(d);
  if (c.sa_k == 1 && c.sa_m != 1 && c.sb_k == 1 && c.sb_n != 1) return false;  // both k-contiguous: no such loop
  if (d->alpha_ptr) return false;
  const uint64_t mask = elem_size(d->dtype) == 8 ? ~0ull : 0xffffffffull;
  return ((d->alpha.bits ^ d->mult_identity.bits) & mask) == 0;
}

// ... and worth it: the plain tiles would leave a good part of their last round of 512 places empty, and every
// workgroup's share of the k-tiles is long enough to carry a tile's prologue and fold
// 70 % or more of the compute units get one tile each and none gets two: the plain direct tile then beats both the
// shared tiles, whose folds cost more than the idle units (2560^3 min-plus: 60 - 66 against 54 - 57 TOPS), and the
// staged tile (2816^3: 71 against 60)
static bool one_tile_each(long long tiles) { return tiles <= 256 && tiles * 10 >= 256 * 7; }

static bool streamk_preferred(const cuasr_amd_srgemm_desc *d, long long batch) {
  if (batch != 1 || d->split_k_slices != 1 || !streamk_usable(d)) return false;
  // min-max and max-min spend two instructions per term and their staged tile is within 5 % of the direct one:
  // the shared tiles' fold costs more than the fuller rounds give (3072^3: 43.7 against 46.6 TOPS; 5120^3 a tie)
  if (d->mult_op == kMinimum || d->mult_op == kMaximum) return false;
  const Problem c = canonical(d);
  const long long tiles = (long long)((c.m + 255) / 256) * ((c.n + 127) / 128), ktiles = (c.k + 15) / 16;
  const long long rounds = (tiles + 511) / 512;
  if (tiles * 10 >= rounds * 512 * 9) return false;   // >= 90 % of the places filled: nothing to gain
  if (d->mult_op == kPlus && one_tile_each(tiles)) return false;   // (the plain tile, one per compute unit: pick_family)
  return tiles >= 64 && tiles * ktiles >= 512 * 48;
}

static int validate(const cuasr_amd_srgemm_desc *d, bool splitk) {
  if (!d) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (d->dtype < CUASR_AMD_F32 || d->dtype > CUASR_AMD_I8) return CUASR_AMD_ERROR_INVALID_DATA_TYPE;
  const int layouts[3] = {d->layout_a, d->layout_b, d->layout_c};
  for (int l : layouts)
    if (l != CUASR_AMD_COLUMN_MAJOR && l != CUASR_AMD_ROW_MAJOR) return CUASR_AMD_ERROR_INVALID_LAYOUT;
  if (!valid_add(d->add_op) || !valid_mult(d->mult_op)) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  const bool fp = d->dtype == CUASR_AMD_F32 || d->dtype == CUASR_AMD_F64 || d->dtype == CUASR_AMD_F16;
  if (fp && (is_bitwise(d->add_op) || is_bitwise(d->mult_op))) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  if (d->m < 0 || d->n < 0 || d->k < 0) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (d->reserved != 0) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (splitk ? d->split_k_slices < 1 : d->split_k_slices != 1) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (d->kernel < CUASR_AMD_KERNEL_AUTO || d->kernel > CUASR_AMD_KERNEL_VALU_STREAMK) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  auto min_ld = [](int layout, int rows, int cols) { return (long long)(layout == CUASR_AMD_COLUMN_MAJOR ? rows : cols); };
  if (d->m > 0 && d->k > 0 && d->lda < min_ld(d->layout_a, d->m, d->k)) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (d->n > 0 && d->k > 0 && d->ldb < min_ld(d->layout_b, d->k, d->n)) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (d->m > 0 && d->n > 0) {
    if (d->ldd < min_ld(d->layout_c, d->m, d->n)) return CUASR_AMD_ERROR_INVALID_PROBLEM;
    if (d->C && d->ldc < min_ld(d->layout_c, d->m, d->n)) return CUASR_AMD_ERROR_INVALID_PROBLEM;
    if (!d->D) return CUASR_AMD_ERROR_INVALID_PROBLEM;
    if (d->k > 0 && (!d->A || !d->B)) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  }
  const size_t es = elem_size(d->dtype), os = operand_size(d->dtype);
  const void *ptrs[4] = {d->C, d->D, d->alpha_ptr, d->beta_ptr};
  for (const void *q : ptrs)
    if (reinterpret_cast<uintptr_t>(q) % es) return CUASR_AMD_ERROR_MISALIGNED_OPERAND;
  if (reinterpret_cast<uintptr_t>(d->A) % os || reinterpret_cast<uintptr_t>(d->B) % os) return CUASR_AMD_ERROR_MISALIGNED_OPERAND;
  if (d->kernel == CUASR_AMD_KERNEL_VALU && !find_valu(d->dtype, d->add_op, d->mult_op))
    return CUASR_AMD_ERROR_NOT_SUPPORTED;
  if (d->kernel == CUASR_AMD_KERNEL_MFMA && !mfma_usable(d)) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  if (d->kernel == CUASR_AMD_KERNEL_VALU_DIRECT && !direct_usable(d)) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  if (d->kernel == CUASR_AMD_KERNEL_VALU_STREAMK && (d->split_k_slices != 1 || !streamk_usable(d))) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  return CUASR_AMD_SUCCESS;
}

static Problem canonical(const cuasr_amd_srgemm_desc *d) {
  Problem p{};
  const long long sa_m = d->layout_a == CUASR_AMD_COLUMN_MAJOR ? 1 : d->lda;
  const long long sa_k = d->layout_a == CUASR_AMD_COLUMN_MAJOR ? d->lda : 1;
  const long long sb_k = d->layout_b == CUASR_AMD_COLUMN_MAJOR ? 1 : d->ldb;
  const long long sb_n = d->layout_b == CUASR_AMD_COLUMN_MAJOR ? d->ldb : 1;
  if (d->layout_c == CUASR_AMD_ROW_MAJOR) {
    p.m = d->m; p.n = d->n;
    p.A = d->A; p.sa_m = sa_m; p.sa_k = sa_k;
    p.B = d->B; p.sb_k = sb_k; p.sb_n = sb_n;
  } else {
    // column-major C: run the transposed problem, C^T = B^T (x) A^T
    p.m = d->n; p.n = d->m;
    p.A = d->B; p.sa_m = sb_n; p.sa_k = sb_k;
    p.B = d->A; p.sb_k = sa_k; p.sb_n = sa_m;
  }
  p.k = d->k;
  p.C = d->C; p.ldc = d->ldc;
  p.D = d->D; p.ldd = d->ldd;
  p.alpha = d->alpha; p.beta = d->beta;
  p.add_identity = d->add_identity; p.mult_identity = d->mult_identity;
  p.alpha_ptr = d->alpha_ptr; p.beta_ptr = d->beta_ptr;
  p.add_op = d->add_op; p.mult_op = d->mult_op;
  p.slices = 1; p.k_per_slice = d->k; p.workspace = nullptr;
  p.batch = 1; p.batch_a = p.batch_b = p.batch_c = p.batch_d = 0;
  return p;
}

enum Family { kNaive = 1, kValu = 2, kMfma = 3, kDirect = 4, kStreamK = 5 };

static int pick_family(const cuasr_amd_srgemm_desc *d, long long batch = 1) {
  if (d->kernel != CUASR_AMD_KERNEL_AUTO) return d->kernel;
  // plus-times is the one semiring a matrix instruction computes as is
  // (its tile is 128 x 128: below 128 tiles half the compute units and more stand idle, and the
  // vector-ALU tiles, which are smaller, are faster -- 1024^3: 31 against 22 TFLOP/s)
  // (binary16: the matrix-core kernel accumulates in float and is not bit-identical to the binary16 sums of the
  // vector-ALU tile and the oracle, so it runs only when the descriptor asks for it)
  if (d->add_op == kPlus && d->mult_op == kMultiplies && d->dtype != CUASR_AMD_F16 && mfma_usable(d)) {
    const long long mfma_tiles = (long long)((d->m + 127) / 128) * ((d->n + 127) / 128) * d->split_k_slices * batch;
    if (mfma_tiles >= 128 || !find_valu(d->dtype, d->add_op, d->mult_op)) return kMfma;
  }
  // On gfx950 the fp32 matrix instructions and the vector ALU share one
  // pipeline, so the matrix-core assisted tropical tile is no faster than the
  // vector-ALU tile; it stays selectable but is not the default.
  // The direct-to-LDS tile is 256 x 128 (128 x 128 when both operands are k-contiguous, and
  // for double) and the chip holds 512 of them at a time (two per compute unit).  It is the fastest family when its workgroups fill
  // whole rounds of 512; a launch that leaves much of a round empty (small or
  // awkwardly sized outputs, split-K of a small output) is better served by the
  // smaller tiles of the staged family, whose many short workgroups balance.
  const Problem c = canonical(d);
  const bool f64 = d->dtype == CUASR_AMD_F64;  // fp64 direct tile: 128 x 128, two per compute unit like the 4-byte one
  const int tile_m = f64 ? 128 : (c.sa_k == 1 && c.sa_m != 1 && c.sb_k == 1 && c.sb_n != 1) ? 128 : 256;  // relaxed variant: 128 x 128
  const int tile_n = 128;
  // (an fp64 instruction occupies the vector ALU for four cycles: one workgroup per compute unit already runs at
  // nearly the full rate -- 2048^3 max-plus, 256 tiles: 30.9 TOPS against 28.8 on the staged tile -- so its rounds are
  // of 256; from `python -m cuasr_amd.bench_matrix --tune`)
  const long long slots = f64 ? 256 : 512;
  const long long direct_groups = (long long)((c.m + tile_m - 1) / tile_m) * ((c.n + tile_n - 1) / tile_n) * d->split_k_slices * batch;
  const long long rounds = (direct_groups + slots - 1) / slots;
  // >= 7/8 of its rounds (fp64: 95 % -- its staged tile is within 10 % of the direct one, so a last round that
  // is 11 % empty, 5120^2, already costs more than the direct tile gains: 28.3 against 29.5 TOPS)
  const bool fills = f64 ? direct_groups * 100 >= rounds * slots * 95 : direct_groups * 8 >= rounds * slots * 7;
  const bool have_valu = find_valu(d->dtype, d->add_op, d->mult_op) != nullptr;
  // or-and: the staged tile turns its panels into masks on their way to LDS and spends one
  // `acc | (a & b)` per term; the direct tile cannot (its panels never pass through registers)
  const bool masked = d->add_op == kLogicalOr && d->mult_op == kLogicalAnd;
  // both operands k-contiguous, 4-byte types: the direct tile has no hand-scheduled loop for that pair of
  // panel forms (two k-quad operands do not fit 128 registers) and its 2-wave variant is slower than the
  // staged tile (4096^3 min-plus: 70.4 against 72.9 TOPS)
  // (float only: on the integer types the 2-wave direct tile wins that case -- xor-and / or-and on words 87 - 88
  // against 77 TOPS at 4096^3, min-plus 47.7 against 45.1, plus-times 45.9 against 41.8)
  const bool kc2 = c.sa_k == 1 && c.sa_m != 1 && c.sb_k == 1 && c.sb_n != 1;
  const bool both_kc = d->dtype == CUASR_AMD_F32 && kc2;
  // integer plus-times on the 4-wave direct tile is a compiled multiply-add loop that spills: 22.6 against 41.9 TOPS
  // on the staged tile (4096^3); its 2-wave form for two k-contiguous operands does not
  const bool slow_direct = (d->dtype == CUASR_AMD_I32 || d->dtype == CUASR_AMD_U32) && d->add_op == kPlus &&
                           d->mult_op == kMultiplies && !kc2;
  if (streamk_preferred(d, batch)) return kStreamK;
  // min-plus / max-plus, which would otherwise share their tiles out (measured for those only: generalised to every
  // pair and type, the rule lost as often as it won; xor-and on words at 2560^3: 63 against 66 TOPS on the staged tile)
  if (batch == 1 && d->split_k_slices == 1 && streamk_usable(d) && d->mult_op == kPlus &&
      one_tile_each((long long)((c.m + 255) / 256) * ((c.n + 127) / 128)))
    return kDirect;
  if (direct_usable(d) && ((fills && !((both_kc || masked || slow_direct) && have_valu)) || !have_valu)) return kDirect;
  if (have_valu) return kValu;
  if (mfma_usable(d)) return kMfma;
  return kNaive;
}

// A large output whose direct-to-LDS tiles do not fill whole rounds (5120^2 is 800 tiles: a round
// and a half) need not give the fast tile up altogether: the largest top-left block of whole tiles
// that does fill its rounds runs on the direct tile, and the strips to its right and below it on
// the staged family.  The three launches write disjoint parts of D and read A, B, C only.
struct Block { int rows, cols; };
static Block direct_block(const cuasr_amd_srgemm_desc *d, const Problem &c) {
  const Block none{0, 0};
  if (d->kernel != CUASR_AMD_KERNEL_AUTO || d->split_k_slices != 1 || !direct_usable(d)) return none;
  if (!find_valu(d->dtype, d->add_op, d->mult_op)) return none;
  const bool f64 = d->dtype == CUASR_AMD_F64;
  // or-and and 4-byte operands that are both k-contiguous prefer the staged tile at any size (pick_family)
  if (d->add_op == kLogicalOr && d->mult_op == kLogicalAnd) return none;
  if (!f64 && c.sa_k == 1 && c.sa_m != 1 && c.sb_k == 1 && c.sb_n != 1) return none;
  // ... and so does integer plus-times (the direct tile's compiled multiply-add loop is the slower one)
  if ((d->dtype == CUASR_AMD_I32 || d->dtype == CUASR_AMD_U32) && d->add_op == kPlus && d->mult_op == kMultiplies) return none;
  const int tile_m = f64 ? 128 : 256;
  const int tile_n = 128;
  const long long slots = 512;
  const int tr = c.m / tile_m, tc = c.n / tile_n;  // whole tiles only
  // fp64: the strips of a mid-sized output are short launches that cost what the block gains (3072^2: 29.0 against
  // 30.8 TOPS on the staged tile alone; 5120^2: 30.6 against 29.5)
  if (f64 && (long long)tr * tc < 1024) return none;
  long long best = 0;
  Block b = none;
  for (int r = 1; r <= tr; ++r) {
    for (int q = tc; q >= 1; --q) {
      const long long t = (long long)r * q;
      if (t <= best) break;  // narrower blocks of this height are smaller still
      const long long rounds = (t + slots - 1) / slots;
      if (t * 100 >= rounds * slots * 97) {
        best = t;
        b = Block{r * tile_m, q * tile_n};
        break;
      }
    }
  }
  // worth three launches only when the block is most of the output
  if (best * tile_m * tile_n * 10 < (long long)c.m * c.n * 6) return none;
  return b;
}

// rows [r0, r0 + rows) x columns [c0, c0 + cols) of the output as a problem of its own
static Problem sub_problem(const Problem &p, size_t es, int r0, int c0, int rows, int cols) {
  Problem q = p;
  q.m = rows;
  q.n = cols;
  q.A = static_cast<const char *>(p.A) + (long long)r0 * p.sa_m * (long long)es;
  q.B = static_cast<const char *>(p.B) + (long long)c0 * p.sb_n * (long long)es;
  if (p.C) q.C = static_cast<const char *>(p.C) + ((long long)r0 * p.ldc + c0) * (long long)es;
  q.D = static_cast<char *>(p.D) + ((long long)r0 * p.ldd + c0) * (long long)es;
  return q;
}

// compute units of the current device (asked once per device)
static int compute_units(void) {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> table[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 0;
  int n = table[dev].load(std::memory_order_relaxed);
  if (n <= 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    table[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

static launch_fn family_fn(int family, const cuasr_amd_srgemm_desc *d) {
  switch (family) {
    case kMfma: return find_mfma(d->dtype, d->add_op, d->mult_op);
    case kDirect: return find_direct(d->dtype, d->add_op, d->mult_op);
    case kValu: return find_valu(d->dtype, d->add_op, d->mult_op);
    default: return find_naive(d->dtype);
  }
}

// Which family a strided batch runs on, and whether the product index goes into the grid (one launch for
// the whole batch) or the batch becomes a sequence of launches.  -1: the descriptor names the direct-to-LDS
// tile and the batch strides do not keep its 16-byte alignment.
static int batched_family(const cuasr_amd_srgemm_desc *desc, int batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                          int64_t stride_d, bool *in_grid_out) {
  const bool col = desc->layout_c == CUASR_AMD_COLUMN_MAJOR;
  int family = pick_family(desc, batch);
  if (family == kDirect && batch > 1) {
    // the direct-to-LDS tiles fetch 16-byte vectors: a batch stride that is no multiple of 16 bytes leaves the
    // later products misaligned; the staged tile takes any element alignment, with the batch still in the grid
    Problem probe = canonical(desc);
    probe.batch = batch < 65535 ? batch : 65535;
    probe.batch_a = col ? stride_b : stride_a;
    probe.batch_b = col ? stride_a : stride_b;
    probe.batch_c = stride_c;
    probe.batch_d = stride_d;
    if (!(desc->dtype == CUASR_AMD_F64 ? direct64_can_run(probe) : direct_can_run(probe))) {
      if (desc->kernel == CUASR_AMD_KERNEL_VALU_DIRECT) return -1;  // asked for by name
      family = find_valu(desc->dtype, desc->add_op, desc->mult_op) ? kValu : kNaive;
    }
  }
  bool in_grid = (family == kValu || family == kDirect) && batch > 1;
  if (family == kMfma && batch > 1 && desc->add_op == kPlus && desc->mult_op == kMultiplies) {
    // the hand-scheduled matrix-core tiles take a batch in the grid too; the compiled ones (ragged k, unaligned
    // products) do not: ask with the first launch's problem
    Problem probe = canonical(desc);
    probe.batch = batch < 65535 ? batch : 65535;
    probe.batch_a = col ? stride_b : stride_a;
    probe.batch_b = col ? stride_a : stride_b;
    in_grid = (desc->dtype == CUASR_AMD_I8 || desc->dtype == CUASR_AMD_F16) ? true : desc->dtype == CUASR_AMD_F64 ? mfma_direct_f64_can_run(probe) : mfma_direct_f32_can_run(probe);
  }
  *in_grid_out = in_grid;
  return family;
}

}  // namespace cuasr_amd

using namespace cuasr_amd;

extern "C" {

int cuasr_amd_abi_version(void) { return CUASR_AMD_ABI_VERSION; }

const char *cuasr_amd_status_string(int status) {
  switch (status) {
    case CUASR_AMD_SUCCESS: return "success";
    case CUASR_AMD_ERROR_MISALIGNED_OPERAND: return "misaligned operand";
    case CUASR_AMD_ERROR_INVALID_DATA_TYPE: return "invalid data type";
    case CUASR_AMD_ERROR_INVALID_LAYOUT: return "invalid layout";
    case CUASR_AMD_ERROR_INVALID_PROBLEM: return "invalid problem";
    case CUASR_AMD_ERROR_NOT_SUPPORTED: return "not supported";
    case CUASR_AMD_ERROR_WORKSPACE_NULL: return "workspace is null";
    case CUASR_AMD_ERROR_INTERNAL: return "internal error";
    case CUASR_AMD_ERROR_ARCH_MISMATCH: return "architecture mismatch";
    case CUASR_AMD_ERROR_INSUFFICIENT_DRIVER: return "insufficient driver";
    case CUASR_AMD_ERROR_MEMORY_ALLOCATION: return "memory allocation failed (or: larger than the library's fixed workspace)";
    default: return "invalid status";
  }
}

int cuasr_amd_srgemm_can_implement(const cuasr_amd_srgemm_desc *desc) { return validate(desc, false); }

const char *cuasr_amd_selected_kernel(const cuasr_amd_srgemm_desc *desc) {
  if (validate(desc, true) != CUASR_AMD_SUCCESS) return nullptr;
  switch (pick_family(desc)) {
    case kMfma: return "mfma";
    case kDirect: return "valu_direct";
    case kStreamK: return "valu_streamk";
    case kValu: return direct_block(desc, canonical(desc)).rows ? "valu_direct+valu" : "valu";  // a block + two strips
    default: return "naive";
  }
}

const char *cuasr_amd_selected_kernel_batched(const cuasr_amd_srgemm_desc *desc, int batch, int64_t stride_a, int64_t stride_b,
                                              int64_t stride_c, int64_t stride_d) {
  if (!desc || batch < 1 || stride_a < 0 || stride_b < 0 || stride_c < 0 || stride_d < 0) return nullptr;
  if (validate(desc, false) != CUASR_AMD_SUCCESS) return nullptr;
  bool in_grid = false;
  switch (batched_family(desc, batch, stride_a, stride_b, stride_c, stride_d, &in_grid)) {
    case kMfma: return in_grid ? "mfma" : "mfma, a launch per product";
    case kDirect: return in_grid ? "valu_direct" : "valu_direct, a launch per product";
    case kValu: return in_grid ? "valu" : "valu, a launch per product";
    case -1: return nullptr;
    default: return "a launch per product";   // each product picks for itself (cuasr_amd_selected_kernel)
  }
}

int cuasr_amd_srgemm(const cuasr_amd_srgemm_desc *desc, void *stream) {
  const int st = validate(desc, false);
  if (st != CUASR_AMD_SUCCESS) return st;
  const Problem p = canonical(desc);
  const int family = pick_family(desc);
  const launch_fn fn = family == kStreamK ? find_direct(desc->dtype, desc->add_op, desc->mult_op) : family_fn(family, desc);
  if (!fn) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (family == kStreamK) {
    // the source term into D, then the product folded into it by two workgroups per compute unit
    const prepare_fold_fn prepare = find_prepare_fold(desc->dtype);
    const streamk_fn run = find_streamk(desc->dtype, desc->add_op, desc->mult_op);
    const int groups = 2 * compute_units();
    if (!prepare || !run || groups <= 0) return CUASR_AMD_ERROR_NOT_SUPPORTED;
    const long long tiles = (long long)((p.m + 255) / 256) * ((p.n + 127) / 128);  // the direct tile is 256 x 128
    if (prepare(p, 256, 128, tiles / groups * groups, s) != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
    return run(p, groups, s) == hipSuccess ? CUASR_AMD_SUCCESS : CUASR_AMD_ERROR_INTERNAL;
  }
  if (family == kValu) {
    const Block b = direct_block(desc, p);
    const launch_fn direct = b.rows ? find_direct(desc->dtype, desc->add_op, desc->mult_op) : nullptr;
    if (direct) {
      const size_t es = elem_size(desc->dtype);
      hipError_t e = direct(sub_problem(p, es, 0, 0, b.rows, b.cols), s);
      if (e == hipSuccess && b.cols < p.n) e = fn(sub_problem(p, es, 0, b.cols, b.rows, p.n - b.cols), s);
      if (e == hipSuccess && b.rows < p.m) e = fn(sub_problem(p, es, b.rows, 0, p.m - b.rows, p.n), s);
      return e == hipSuccess ? CUASR_AMD_SUCCESS : CUASR_AMD_ERROR_INTERNAL;
    }
  }
  return fn(p, s) == hipSuccess ? CUASR_AMD_SUCCESS : CUASR_AMD_ERROR_INTERNAL;
}

// A strided batch.  The tile kernels -- the vector-ALU ones and the hand-scheduled matrix-core ones -- take the
// product index from the grid (blockIdx.z), so a batch of small products is one launch that fills the chip; the
// compiled matrix-core kernels (ragged k, unaligned products) and the naive kernel, and batches beyond the
// grid's 65535, are sequences of launches.
int cuasr_amd_srgemm_batched(const cuasr_amd_srgemm_desc *desc, int batch, int64_t stride_a, int64_t stride_b,
                             int64_t stride_c, int64_t stride_d, void *stream) {
  if (!desc || batch < 0 || stride_a < 0 || stride_b < 0 || stride_c < 0 || stride_d < 0)
    return CUASR_AMD_ERROR_INVALID_PROBLEM;
  const int st = validate(desc, false);
  if (st != CUASR_AMD_SUCCESS) return st;
  // the outputs must not overlap: at least the span of one matrix apart
  const bool col = desc->layout_c == CUASR_AMD_COLUMN_MAJOR;
  const int64_t outer = col ? desc->n : desc->m, inner = col ? desc->m : desc->n;
  if (batch > 1 && outer > 0 && inner > 0 && stride_d < (outer - 1) * desc->ldd + inner) return CUASR_AMD_ERROR_INVALID_PROBLEM;
  if (batch == 0) return CUASR_AMD_SUCCESS;
  const int64_t es = int64_t(elem_size(desc->dtype)), os = int64_t(operand_size(desc->dtype));
  bool in_grid = false;
  const int family = batched_family(desc, batch, stride_a, stride_b, stride_c, stride_d, &in_grid);
  if (family < 0) return CUASR_AMD_ERROR_MISALIGNED_OPERAND;  // the direct-to-LDS tile asked for by name, strides off 16 bytes
  if (in_grid) {
    const launch_fn fn = family_fn(family, desc);
    if (!fn) return CUASR_AMD_ERROR_NOT_SUPPORTED;
    Problem p = canonical(desc);
    // a column-major output runs as the transposed problem: the roles of A and B swap, and so do their strides
    p.batch_a = col ? stride_b : stride_a;
    p.batch_b = col ? stride_a : stride_b;
    p.batch_c = stride_c;
    p.batch_d = stride_d;
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (int first = 0; first < batch; first += 65535) {
      p.batch = batch - first < 65535 ? batch - first : 65535;
      if (fn(p, s) != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
      p.A = static_cast<const char *>(p.A) + os * p.batch_a * p.batch;
      p.B = static_cast<const char *>(p.B) + os * p.batch_b * p.batch;
      if (p.C) p.C = static_cast<const char *>(p.C) + es * p.batch_c * p.batch;
      p.D = static_cast<char *>(p.D) + es * p.batch_d * p.batch;
    }
    return CUASR_AMD_SUCCESS;
  }
  for (int i = 0; i < batch; ++i) {
    cuasr_amd_srgemm_desc one = *desc;
    if (one.A) one.A = static_cast<const char *>(desc->A) + os * stride_a * i;
    if (one.B) one.B = static_cast<const char *>(desc->B) + os * stride_b * i;
    if (one.C) one.C = static_cast<const char *>(desc->C) + es * stride_c * i;
    if (one.D) one.D = static_cast<char *>(desc->D) + es * stride_d * i;
    const int r = cuasr_amd_srgemm(&one, stream);
    if (r != CUASR_AMD_SUCCESS) return r;
  }
  return CUASR_AMD_SUCCESS;
}

size_t cuasr_amd_splitk_workspace_bytes(const cuasr_amd_srgemm_desc *desc) {
  if (!desc || desc->m < 0 || desc->n < 0 || desc->split_k_slices < 1) return 0;
  if (desc->dtype < CUASR_AMD_F32 || desc->dtype > CUASR_AMD_I8) return 0;
  return elem_size(desc->dtype) * size_t(desc->m) * size_t(desc->n) * size_t(desc->split_k_slices);
}

// fills `count` 4-byte words with `bits` (a plain kernel rather than a memset node: this may run under stream capture)
static __global__ __launch_bounds__(256) void fill_words_kernel(uint32_t *dst, long long count, uint32_t bits) {
  const long long i = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 4 <= count) {
    *reinterpret_cast<uint4 *>(dst + i) = make_uint4(bits, bits, bits, bits);
  } else {
    for (long long j = i; j < count; ++j) dst[j] = bits;
  }
}

// Split-K of a small output on the staged tiles: how many workgroups share one slice's k range (Problem::k_sub).
// The quarter-size tile runs with four groups of waves per workgroup, one workgroup per compute unit; fewer than
// half as many (tile, slice) pairs as compute units leave the rest of the chip idle (256 x 256 x 65536 in 8
// slices: 128 workgroups, 31.9 TOPS against 51.5 in 16 slices).  Only where the parts can meet through native
// atomics (4-byte minimum / maximum, or / xor on words) and every part keeps a long run of k-tiles.
static int sub_slices(const cuasr_amd_srgemm_desc *d, const Problem &p, int units) {
  if (units <= 0 || p.batch != 1 || p.slices < 1) return 1;
  const bool fp = d->dtype == CUASR_AMD_F32;
  if (!fp && d->dtype != CUASR_AMD_I32 && d->dtype != CUASR_AMD_U32) return 1;
  const bool minmax = d->add_op == kMinimum || d->add_op == kMaximum;
  if (!(minmax || (!fp && (d->add_op == kBitOr || d->add_op == kBitXor)))) return 1;
  if (fp && d->mult_op == kMultiplies) return 1;   // a zero result's sign depends on the whole k range
  if (reinterpret_cast<uintptr_t>(p.workspace) % 16) return 1;
  const long long groups = (long long)((p.m + 63) / 64) * ((p.n + 63) / 64) * p.slices;
  if (groups * 2 > units) return 1;
  long long sub = units / groups;
  const long long max_sub = p.k_per_slice / 1024;   // at least 32 k-tiles of 32 per part
  if (sub > max_sub) sub = max_sub;
  return sub >= 2 ? (int)sub : 1;
}

// Both split-K forms: partial products of the K-slices into the workspace, then one
// reduction kernel (`serial` picks the ordered replay of the serial form's epilogues).
// `stages`: 1 = the slice kernel, 2 = the reduction kernel, 3 = both.
static int run_splitk(const cuasr_amd_srgemm_desc *desc, void *workspace, void *stream, bool serial, int stages = 3) {
  const int st = validate(desc, true);
  if (st != CUASR_AMD_SUCCESS) return st;
  if (!workspace) return CUASR_AMD_ERROR_WORKSPACE_NULL;
  if (reinterpret_cast<uintptr_t>(workspace) % elem_size(desc->dtype)) return CUASR_AMD_ERROR_MISALIGNED_OPERAND;
  Problem p = canonical(desc);
  p.slices = desc->split_k_slices;
  // slice extent: whole k-tiles, spread evenly; trailing slices may be empty and then
  // hold the additive identity.  The serial form's result can depend on where the
  // slices end (alpha multiplies every partial), so it keeps the reference's extent,
  // ceil(ceil(K / 8) / S) * 8 (include/cuasr/gemm/kernel/srgemm.h:97-100); the parallel
  // form's cannot, beyond the rounding of sums, and uses this library's k-tile of 16.
  const int tile = serial ? 8 : 16;
  const long long tiles = (p.k + tile - 1) / tile;
  const long long per = (tiles + p.slices - 1) / p.slices;
  p.k_per_slice = int(per * tile > 0 ? per * tile : tile);
  p.workspace = workspace;
  // The direct-to-LDS tiles store partial tiles as 16-byte vectors; family selection looks at the
  // operands only, so a workspace that is element-aligned but not 16-byte aligned is sorted out here:
  // AUTO goes on to the staged family (or the naive kernel), a forced direct tile is refused.
  int family = pick_family(desc);
  if (family == kStreamK) family = kDirect;  // (one slice through the split-K entry points: the plain tile)
  if (family == kDirect && !(desc->dtype == CUASR_AMD_F64 ? direct64_can_run(p) : direct_can_run(p))) {
    if (desc->kernel != CUASR_AMD_KERNEL_AUTO) return CUASR_AMD_ERROR_MISALIGNED_OPERAND;
    family = find_valu(desc->dtype, desc->add_op, desc->mult_op) ? kValu : kNaive;
  }
  const launch_fn fn = family_fn(family, desc);
  const launch_fn red = serial ? find_reduce_serial(desc->dtype) : find_reduce(desc->dtype);
  if (!fn || !red) return CUASR_AMD_ERROR_NOT_SUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if ((stages & 1) && family == kValu && desc->kernel != CUASR_AMD_KERNEL_NAIVE) {
    p.k_sub = sub_slices(desc, p, compute_units());
    if (p.k_sub > 1) {
      // the parts of a slice fold into its partial tile: start every partial tile at the additive identity
      const long long words = (long long)p.m * p.n * p.slices;
      fill_words_kernel<<<dim3((unsigned)((words + 1023) / 1024)), dim3(256), 0, s>>>(static_cast<uint32_t *>(workspace), words, p.add_identity.u32);
      if (hipGetLastError() != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
    }
  }
  if ((stages & 1) && fn(p, s) != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
  if ((stages & 2) && red(p, s) != hipSuccess) return CUASR_AMD_ERROR_INTERNAL;
  return CUASR_AMD_SUCCESS;
}

int cuasr_amd_srgemm_splitk(const cuasr_amd_srgemm_desc *desc, void *workspace, void *stream) {
  return run_splitk(desc, workspace, stream, false);
}

int cuasr_amd_reduce_splitk(const cuasr_amd_srgemm_desc *desc, void *workspace, void *stream) {
  return run_splitk(desc, workspace, stream, false, 2);
}

// ---- split-K for callers that cannot allocate: the workspace is a fixed array in the library's
// own device image, one copy per GPU, shared by every call on that GPU.
static __device__ __align__(256) unsigned char scratch[CUASR_AMD_STATIC_WORKSPACE_BYTES];

// Device address of `scratch` on the current GPU.  The array's name is only a host-side handle
// for the symbol; the address is asked for once per device, with that device current, and kept.
static void *static_workspace(void) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void *> table[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void *ptr = table[dev].load(std::memory_order_acquire);
  if (!ptr) {
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return nullptr;
    table[dev].store(ptr, std::memory_order_release);  // every thread finds the same address
  }
  return ptr;
}

int cuasr_amd_srgemm_splitk_static(const cuasr_amd_srgemm_desc *desc, void *stream) {
  const int st = validate(desc, true);
  if (st != CUASR_AMD_SUCCESS) return st;
  // the partial tiles of all slices must fit (no overflow: m * n < 2^62, and the quotient bounds the rest)
  const unsigned long long elems = (unsigned long long)desc->m * (unsigned long long)desc->n;
  const unsigned long long room = CUASR_AMD_STATIC_WORKSPACE_BYTES / elem_size(desc->dtype);
  if (elems > room || elems * (unsigned long long)desc->split_k_slices > room) return CUASR_AMD_ERROR_MEMORY_ALLOCATION;
  void *ws = static_workspace();
  if (!ws) return CUASR_AMD_ERROR_INTERNAL;
  // nothing in the array has to start at zero: the slice kernels write every element of the
  // slices the reduction reads (empty trailing slices are filled with the additive identity)
  return run_splitk(desc, ws, stream, false);
}

size_t cuasr_amd_splitk_serial_workspace_bytes(const cuasr_amd_srgemm_desc *desc) {
  if (!desc || desc->split_k_slices <= 1) return 0;
  return cuasr_amd_splitk_workspace_bytes(desc);
}

int cuasr_amd_srgemm_splitk_serial(const cuasr_amd_srgemm_desc *desc, void *workspace, void *stream) {
  if (desc && desc->split_k_slices == 1) return cuasr_amd_srgemm(desc, stream);  // no workspace, no reduction
  return run_splitk(desc, workspace, stream, true);
}

}  // extern "C"
