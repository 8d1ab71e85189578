"""Half precision (binary16 in every operand and the accumulator) against the CPU oracle, bit for bit,
through the C ABI: the packed vector-ALU tile in both its forms (whole tiles of aligned operands, and
guarded), every layout, the naive kernel for the pairs the tile does not take, split-K, batches, views."""
import numpy as np
import pytest

from helpers import assert_same_bits, order_of, to_device

pytestmark = pytest.mark.gpu

TILE_PAIRS = [("minimum", "plus"), ("maximum", "plus"), ("minimum", "maximum"), ("maximum", "minimum"), ("plus", "multiplies"),
              ("minimum", "multiplies"), ("maximum", "multiplies"), ("logical_or", "logical_and")]
OTHER_PAIRS = [("plus", "maximum"), ("logical_or", "plus")]     # (pairs no tile serves: the naive kernel)
LAYOUTS = ["ccc", "rrr", "crc", "rcr", "rcc", "crr", "ccr", "rrc"]


def operands(add, mult, m, n, k, la, lb, lc, seed=1):
    """Values whose sums and products do not fit binary16 exactly, so that every operator's rounding counts."""
    from cuasr_amd import inputs
    lo, hi = (-1.0, 1.0) if mult == "multiplies" else (0.5, 100.0)
    A = inputs.uniform(seed, m, k, lo, hi, np.float16, order_of(la))
    B = inputs.uniform(seed + 1, k, n, lo, hi, np.float16, order_of(lb))
    C = inputs.uniform(seed + 2, m, n, lo, hi, np.float16, order_of(lc))
    if mult == "logical_and":
        A[A < 97] = 0          # sparse, and zeros of both signs: -0 is false as well
        B[B < 97] = 0
        A[::3, ::5] = np.float16(-0.0)
    return A, B, C


def scalars(add, mult, beta_one):
    import cuasr_amd
    ident = cuasr_amd.op_identity(add, "f16", True)
    one = cuasr_amd.op_identity(mult, "f16", True)
    zero = cuasr_amd.op_annihilator(mult, "f16", True)
    if add == "maximum" and mult == "plus":
        zero = ident  # the max-semiring zero, not plus::Annihilator
    return ident, one, (one if beta_one else zero)


def check(oracle, add, mult, m, n, k, layouts, kernel, beta_one=True, seed=1, splitk=0, alpha=None, beta=None):
    import torch
    import cuasr_amd
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    A, B, C = operands(add, mult, m, n, k, la, lb, lc, seed)
    ident, one, b = scalars(add, mult, beta_one)
    alpha = one if alpha is None else np.float16(alpha)
    beta = b if beta is None else np.float16(beta)
    want = oracle.srgemm(add, mult, A, B, C, alpha, beta, ident)   # (split-K runs order-free adds only: the slices cannot matter)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD = to_device(np.zeros_like(C))
    print(f"half {add}-{mult} {m}x{n}x{k} {layouts} {kernel} beta_one={beta_one} splitk={splitk}", flush=True)
    if splitk:
        ws = torch.empty(cuasr_amd.splitk_workspace_bytes(m, n, splitk, "f16") // 2 + 8, dtype=torch.float16, device="cuda")
        cuasr_amd.srgemm_splitk(add, mult, dA, dB, dC, dD, splitk, ws, alpha, beta, ident, one, dtype="f16", kernel=kernel)
    else:
        cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, alpha, beta, ident, one, dtype="f16", kernel=kernel)
    torch.cuda.synchronize()
    assert_same_bits(dD.cpu().numpy(), want, f"{add}-{mult} f16 {m}x{n}x{k} {layouts} {kernel}")


@pytest.mark.parametrize("sr", TILE_PAIRS)
@pytest.mark.parametrize("layouts", LAYOUTS)
def test_packed_tile(oracle, lib, sr, layouts):
    # whole tiles (the unguarded kernel), ragged everything, single element, tall and thin
    for shape in [(128, 256, 32), (256, 512, 96), (100, 300, 45), (1, 1, 1), (130, 258, 33), (64, 8, 200)]:
        for beta_one in (False, True):
            check(oracle, *sr, *shape, layouts, "valu", beta_one)


@pytest.mark.parametrize("layouts", LAYOUTS)
def test_every_tile_size(oracle, lib, layouts):
    """The kernel comes in three tile sizes, picked by how many workgroups the output gives the chip: the full
    tile unguarded (whole tiles of aligned operands) and guarded, the 64 x 128 tile, the 32 x 128 tile."""
    check(oracle, "minimum", "plus", 4096, 4096, 64, layouts, "valu")              # 512 full tiles, unguarded
    check(oracle, "maximum", "minimum", 4000, 4100, 70, layouts, "valu", False)    # full tiles, ragged: guarded
    check(oracle, "minimum", "plus", 2048, 2048, 96, layouts, "valu")              # 64 x 128 tiles
    check(oracle, "plus", "multiplies", 1000, 2000, 50, layouts, "valu")           # 64 x 128 tiles, ragged
    check(oracle, "maximum", "plus", 1536, 1536, 64, layouts, "valu")              # 32 x 128 tiles, k shared out between the waves
    check(oracle, "maximum", "plus", 1024, 1024, 64, layouts, "valu")              # 16 x 128 tiles, likewise
    check(oracle, "plus", "multiplies", 1024, 1024, 64, layouts, "valu")           # 32 x 128 tiles, whole k-tiles per thread


@pytest.mark.parametrize("sr", [x for x in TILE_PAIRS if x[0] != "plus"])
@pytest.mark.parametrize("layouts", ["ccc", "rcr", "crr", "rrc"])
def test_k_shared_out_between_waves(oracle, lib, sr, layouts):
    """The two small tiles of the order-free adds: each wave takes a quarter of every k-tile and the four partial
    accumulators meet in LDS.  k that ends inside the first, second, third, fourth quarter of a tile; one tile; k
    shorter than a quarter; extents that are no multiple of anything; and the split-K forms on top."""
    for k in (3, 9, 17, 31, 32, 45, 64, 250):
        check(oracle, *sr, 520, 390, k, layouts, "valu", beta_one=bool(k & 1))       # 16 x 128 tiles
    check(oracle, *sr, 1530, 1300, 77, layouts, "valu")                             # 32 x 128 tiles
    check(oracle, *sr, 1530, 1300, 32, layouts, "valu", beta_one=False)
    check(oracle, *sr, 300, 260, 500, layouts, "valu", splitk=5)


def test_selected_family(lib):
    import cuasr_amd
    dA = to_device(np.zeros((128, 64), np.float16))
    dB = to_device(np.zeros((64, 256), np.float16))
    dD = to_device(np.zeros((128, 256), np.float16))
    for (add, mult), name in [(("minimum", "plus"), b"valu"), (("plus", "multiplies"), b"valu"), (("minimum", "multiplies"), b"valu"),
                              (("logical_or", "logical_and"), b"valu"), (("plus", "maximum"), b"naive")]:
        ident, one, zero = scalars(add, mult, False)
        desc = cuasr_amd.make_desc(add, mult, "f16", dA, dB, dD, dD, one, zero, ident, one)
        assert lib.cuasr_amd_selected_kernel(desc) == name
    # bitwise operators are not defined on floating point
    desc = cuasr_amd.make_desc("bit_xor", "bit_and", "f16", dA, dB, dD, dD, 0, 0, 0, 1)
    assert lib.cuasr_amd_srgemm_can_implement(desc) == 5


@pytest.mark.parametrize("sr", TILE_PAIRS + OTHER_PAIRS)
@pytest.mark.parametrize("kernel", ["auto", "naive"])
def test_every_pair(oracle, lib, sr, kernel):
    for layouts in ("ccc", "rcr"):
        check(oracle, *sr, 70, 90, 33, layouts, kernel)
        check(oracle, *sr, 128, 256, 64, layouts, kernel, beta_one=False)


@pytest.mark.parametrize("layouts", ["ccc", "rcr", "crr", "rrc"])
def test_boolean_closure_on_masks(oracle, lib, layouts):
    """or-and (functional.h:212, :252): the tile works on 16-bit masks; sparse operands so that the answer is
    not all ones, every tile size, an identity that is not zero, alpha / beta that are zero or not."""
    check(oracle, "logical_or", "logical_and", 1024, 1024, 64, layouts, "valu")      # 32 x 128 tiles
    check(oracle, "logical_or", "logical_and", 2048, 2048, 40, layouts, "valu")      # 64 x 128 tiles
    check(oracle, "logical_or", "logical_and", 4096, 4096, 32, layouts, "valu")      # full tiles, unguarded
    check(oracle, "logical_or", "logical_and", 4000, 4100, 37, layouts, "valu", beta_one=False)
    check(oracle, "logical_or", "logical_and", 300, 200, 45, layouts, "valu", alpha=0.0, beta=2.5)
    check(oracle, "logical_or", "logical_and", 300, 200, 45, layouts, "valu", alpha=-3.0, beta=0.0)


@pytest.mark.parametrize("add", ["minimum", "maximum"])
@pytest.mark.parametrize("layouts", ["ccc", "rcr", "crr"])
def test_sign_of_a_zero_extremum(oracle, lib, add, layouts):
    """min-times / max-times whose result is a zero: the reference's comparison keeps the newer of two equal
    operands, so the zero carries the sign of the last zero product of the k range.  Operands drawn from
    {+0, -0} and values of one sign make every result such a zero or a proper extremum."""
    import torch
    import cuasr_amd
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    rng = np.random.default_rng(17)
    sign = 1.0 if add == "minimum" else -1.0          # products are >= 0 (min) or <= 0 (max), zeros of both signs
    # (not through split-K: which zero a split product keeps depends on where the slices end)
    for (m, n, k), slices in [((130, 258, 67), 0), ((64, 128, 40), 0), ((2048, 2048, 40), 0)]:
        A = np.asarray(rng.choice(np.array([0.0, -0.0, 1.0, 2.5], np.float16), (m, k)), order=order_of(la))
        B = np.asarray(rng.choice(np.array([0.0, -0.0, sign * 1.0, sign * 3.0], np.float16), (k, n)), order=order_of(lb))
        C = np.asarray(rng.choice(np.array([0.0, -0.0, sign * 5.0], np.float16), (m, n)), order=order_of(lc))
        ident, one, _ = scalars(add, "multiplies", True)
        want = oracle.srgemm(add, "multiplies", A, B, C, one, one, ident)
        assert (want.view(np.uint16) == 0x8000).any() and (want.view(np.uint16) == 0).any()   # zeros of both signs
        for kernel in ("valu", "naive"):
            dA, dB, dC = to_device(A), to_device(B), to_device(C)
            dD = to_device(np.zeros_like(C))
            if slices:
                ws = torch.empty(m * n * slices + 8, dtype=torch.float16, device="cuda")
                cuasr_amd.srgemm_splitk(add, "multiplies", dA, dB, dC, dD, slices, ws, one, one, ident, one, dtype="f16", kernel=kernel)
            else:
                cuasr_amd.srgemm(add, "multiplies", dA, dB, dC, dD, one, one, ident, one, dtype="f16", kernel=kernel)
            torch.cuda.synchronize()
            assert_same_bits(dD.cpu().numpy(), want, f"{add}-times zeros {m}x{n}x{k} {layouts} {kernel} slices={slices}")


def test_scaled_epilogue(oracle, lib):
    # alpha and beta that are neither identity nor annihilator: both products are rounded before the add
    check(oracle, "plus", "multiplies", 128, 256, 64, "ccc", "valu", alpha=1.5, beta=-0.75)
    check(oracle, "plus", "multiplies", 90, 70, 50, "rcr", "valu", alpha=0.3, beta=2.5)
    check(oracle, "minimum", "plus", 128, 256, 64, "ccc", "valu", alpha=3.25, beta=0.125)
    check(oracle, "maximum", "minimum", 130, 100, 64, "crc", "valu", alpha=40.0, beta=60.0)


@pytest.mark.parametrize("slices", [1, 3, 8])
@pytest.mark.parametrize("kernel", ["auto", "naive"])
def test_splitk(oracle, lib, slices, kernel):
    for shape, layouts in [((256, 256, 1024), "ccc"), ((100, 60, 1000), "rcr"), ((128, 256, 96), "crc")]:
        check(oracle, "minimum", "plus", *shape, layouts, kernel, splitk=slices)
        check(oracle, "maximum", "minimum", *shape, layouts, kernel, splitk=slices, beta_one=False)


def test_apsp_shaped_1024(oracle, lib):
    for layouts in ("ccc", "rcr", "crr"):
        check(oracle, "minimum", "plus", 1024, 1024, 1024, layouts, "auto")
    check(oracle, "plus", "multiplies", 512, 512, 512, "ccc", "auto")


def test_views_at_odd_offsets(oracle, lib):
    """Operands inside larger allocations, two bytes off every vector boundary: the guarded kernel."""
    import torch
    import cuasr_amd
    m, n, k = 131, 257, 67
    for layouts in ("ccc", "rcr"):
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        A, B, C = operands("minimum", "plus", m + 3, n + 3, k + 3, la, lb, lc, seed=9)   # each three larger than its view
        ident, one, _ = scalars("minimum", "plus", True)
        a, b, c = A[1:1 + m, 1:1 + k], B[1:1 + k, 1:1 + n], C[1:1 + m, 1:1 + n]
        want = oracle.srgemm("minimum", "plus", a, b, c, one, one, ident)
        dA, dB, dC = to_device(A), to_device(B), to_device(C)
        dD = to_device(np.full_like(C, 7))
        cuasr_amd.srgemm("minimum", "plus", dA[1:1 + m, 1:1 + k], dB[1:1 + k, 1:1 + n], dC[1:1 + m, 1:1 + n], dD[1:1 + m, 1:1 + n],
                         one, one, ident, one, dtype="f16")
        torch.cuda.synchronize()
        got = dD.cpu().numpy()
        assert_same_bits(got[1:1 + m, 1:1 + n], want, f"view {layouts}")
        frame = got.copy()
        frame[1:1 + m, 1:1 + n] = 7
        assert (frame == 7).all(), "wrote outside the view"


def test_batch_in_the_grid(oracle, lib):
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    for (m, n, k, batch) in [(64, 64, 64, 9), (128, 256, 64, 3), (50, 30, 70, 4)]:
        A = inputs.uniform(3, batch * m, k, 0.5, 100.0, np.float16, "C").reshape(batch, m, k)
        B = inputs.uniform(4, batch * k, n, 0.5, 100.0, np.float16, "C").reshape(batch, k, n)
        C = inputs.uniform(5, batch * m, n, 0.5, 100.0, np.float16, "C").reshape(batch, m, n)
        ident, one, _ = scalars("minimum", "plus", True)
        dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
        dD = torch.zeros_like(dC)
        cuasr_amd.srgemm_batched("minimum", "plus", dA, dB, dC, dD, one, one, ident, one, dtype="f16")
        torch.cuda.synchronize()
        got = dD.cpu().numpy()
        for i in range(batch):
            want = oracle.srgemm("minimum", "plus", A[i], B[i], C[i], one, one, ident)
            assert_same_bits(got[i], want, f"batch product {i} of {m}x{n}x{k}")


@pytest.mark.parametrize("layouts", LAYOUTS)
def test_plus_times_matrix_cores_exact_on_small_integers(oracle, lib, layouts):
    """kernel = mfma on binary16 operands accumulates in float (the reference's ElementAccumulator = float).  On
    small integers every product, every partial sum in either precision and the result are exact, so the output
    must equal the oracle's binary16 sums bit for bit: this checks the fragment layouts, the transposing stager,
    the guards and the epilogue.  Whole tiles (the unguarded kernel), ragged everything, single element, thin."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for (m, n, k), (alpha, beta) in [((128, 128, 64), (1, 0)), ((256, 384, 192), (1, 1)), ((100, 70, 45), (2, -1)), ((1, 1, 1), (1, 1)),
                                     ((130, 258, 67), (-1, 2)), ((64, 8, 200), (1, 1)), ((16, 16, 16), (1, 0)), ((512, 256, 128), (1, 1))]:
        A = inputs.integers(21, m, k, -2, 2, np.float16, order_of(la))
        B = inputs.integers(22, k, n, -2, 2, np.float16, order_of(lb))
        C = inputs.integers(23, m, n, -8, 8, np.float16, order_of(lc))
        want = oracle.srgemm("plus", "multiplies", A, B, C, np.float16(alpha), np.float16(beta), np.float16(0))
        assert np.abs(want.astype(np.float64)).max() <= 2048
        dD = to_device(np.full_like(C, 7))
        print(f"half plus-times mfma {m}x{n}x{k} {layouts} alpha={alpha} beta={beta}", flush=True)
        cuasr_amd.srgemm("plus", "multiplies", to_device(A), to_device(B), to_device(C), dD, np.float16(alpha), np.float16(beta),
                         np.float16(0), np.float16(1), dtype="f16", kernel="mfma")
        torch.cuda.synchronize()
        assert_same_bits(dD.cpu().numpy(), want, f"plus-times f16 mfma {m}x{n}x{k} {layouts}")


@pytest.mark.parametrize("layouts", ["ccc", "rcr", "crr", "rrc"])
def test_plus_times_matrix_cores_float_accumulation(lib, layouts):
    """On data whose sums do not fit binary16, the matrix-core kernel must be within one binary16 rounding of
    alpha * (A B) + beta * C computed in double, plus the error of a float sum: |d - r| <= 2^-11 |r| + 1e-5 sum |a||b|
    (the vector-ALU tile, which rounds every partial sum to binary16, is far outside that bound at k = 1024)."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for (m, n, k) in [(256, 256, 1024), (1000, 900, 333)]:
        A = inputs.uniform(31, m, k, -1.0, 1.0, np.float16, order_of(la))
        B = inputs.uniform(32, k, n, -1.0, 1.0, np.float16, order_of(lb))
        C = inputs.uniform(33, m, n, -4.0, 4.0, np.float16, order_of(lc))
        alpha, beta = np.float16(0.75), np.float16(-1.5)
        r = float(alpha) * (A.astype(np.float64) @ B.astype(np.float64)) + float(beta) * C.astype(np.float64)
        bound = 2.0 ** -11 * np.abs(r) + 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + 1e-7
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm("plus", "multiplies", to_device(A), to_device(B), to_device(C), dD, alpha, beta, np.float16(0), np.float16(1),
                         dtype="f16", kernel="mfma")
        torch.cuda.synchronize()
        err = np.abs(dD.cpu().numpy().astype(np.float64) - r)
        assert (err <= bound).all(), f"{m}x{n}x{k} {layouts}: worst excess {(err - bound).max():.3e}"


def test_matrix_cores_only_on_request(lib):
    """The library's own choice for binary16 plus-times stays the tile that is bit-identical to the oracle; the
    float-accumulating kernel has no split-K form (its partial sums would have to leave as binary16)."""
    import torch
    import cuasr_amd
    dA = to_device(np.zeros((4096, 64), np.float16))
    dB = to_device(np.zeros((64, 4096), np.float16))
    dD = to_device(np.zeros((4096, 4096), np.float16))
    desc = cuasr_amd.make_desc("plus", "multiplies", "f16", dA, dB, dD, dD, 1, 0, 0, 1)
    assert lib.cuasr_amd_selected_kernel(desc) == b"valu"
    desc = cuasr_amd.make_desc("plus", "multiplies", "f16", dA, dB, dD, dD, 1, 0, 0, 1, kernel="mfma")
    assert lib.cuasr_amd_srgemm_can_implement(desc) == 0 and lib.cuasr_amd_selected_kernel(desc) == b"mfma"
    desc = cuasr_amd.make_desc("minimum", "plus", "f16", dA, dB, dD, dD, 0, 0, float("inf"), 0, kernel="mfma")
    assert lib.cuasr_amd_srgemm_can_implement(desc) == 5
    ws = torch.empty(4096 * 4096 * 2, dtype=torch.float16, device="cuda")
    with pytest.raises(cuasr_amd.CuasrError) as e:
        cuasr_amd.srgemm_splitk("plus", "multiplies", dA, dB, dD, dD, 2, ws, 1, 0, 0, 1, dtype="f16", kernel="mfma")
    assert e.value.status == 5


def test_plus_times_matrix_cores_batch_and_views(oracle, lib):
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    for (m, n, k, batch) in [(128, 128, 64, 5), (50, 30, 70, 4)]:
        A = inputs.integers(3, batch * m, k, -2, 2, np.float16, "C").reshape(batch, m, k)
        B = inputs.integers(4, batch * k, n, -2, 2, np.float16, "C").reshape(batch, k, n)
        C = inputs.integers(5, batch * m, n, -8, 8, np.float16, "C").reshape(batch, m, n)
        dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
        dD = torch.zeros_like(dC)
        cuasr_amd.srgemm_batched("plus", "multiplies", dA, dB, dC, dD, np.float16(1), np.float16(1), np.float16(0), np.float16(1), dtype="f16", kernel="mfma")
        torch.cuda.synchronize()
        got = dD.cpu().numpy()
        for i in range(batch):
            want = oracle.srgemm("plus", "multiplies", A[i], B[i], C[i], np.float16(1), np.float16(1), np.float16(0))
            assert_same_bits(got[i], want, f"batch product {i} of {m}x{n}x{k}")
    # operands inside larger allocations, two bytes off every vector boundary
    m, n, k = 131, 257, 67
    for layouts in ("ccc", "rcr"):
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        A = inputs.integers(6, m + 3, k + 3, -2, 2, np.float16, order_of(la))
        B = inputs.integers(7, k + 3, n + 3, -2, 2, np.float16, order_of(lb))
        C = inputs.integers(8, m + 3, n + 3, -8, 8, np.float16, order_of(lc))
        want = oracle.srgemm("plus", "multiplies", A[1:1 + m, 1:1 + k], B[1:1 + k, 1:1 + n], C[1:1 + m, 1:1 + n], np.float16(1), np.float16(1), np.float16(0))
        dA, dB, dC = to_device(A), to_device(B), to_device(C)
        dD = to_device(np.full_like(C, 7))
        cuasr_amd.srgemm("plus", "multiplies", dA[1:1 + m, 1:1 + k], dB[1:1 + k, 1:1 + n], dC[1:1 + m, 1:1 + n], dD[1:1 + m, 1:1 + n],
                         np.float16(1), np.float16(1), np.float16(0), np.float16(1), dtype="f16", kernel="mfma")
        torch.cuda.synchronize()
        got = dD.cpu().numpy()
        assert_same_bits(got[1:1 + m, 1:1 + n], want, f"view {layouts}")
        frame = got.copy()
        frame[1:1 + m, 1:1 + n] = 7
        assert (frame == 7).all(), "wrote outside the view"


def test_no_terms(oracle, lib):
    # k = 0: the accumulator is the additive identity and only the epilogue runs
    check(oracle, "minimum", "plus", 40, 50, 0, "ccc", "auto")
    check(oracle, "plus", "multiplies", 128, 256, 0, "rcr", "valu")


@pytest.mark.parametrize("slices", [1, 2, 5])
def test_serial_splitk(oracle, lib, slices):
    """The serial split-K chain of epilogues in binary16 (small integers: the sums inside a slice are exact in
    any order; alpha multiplies every slice's partial product, as in the reference)."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    for (add, mult, alpha, beta, ident, one), layouts in [(("minimum", "plus", 3.0, 0.0, np.inf, 0.0), "ccc"),
                                                           (("plus", "multiplies", 2.0, -3.0, 0.0, 1.0), "rcr"),
                                                           (("maximum", "minimum", 5.0, np.inf, -np.inf, np.inf), "crc")]:
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        m, n, k = 130, 258, 200
        A = inputs.integers(31, m, k, -4, 4, np.float16, order_of(la))
        B = inputs.integers(1031, k, n, -4, 4, np.float16, order_of(lb))
        C = inputs.integers(2031, m, n, -4, 4, np.float16, order_of(lc))
        f = np.float16
        want = oracle.srgemm_splitk_serial(add, mult, A, B, C, f(alpha), f(beta), f(ident), f(one), slices)
        nbytes = cuasr_amd.splitk_serial_workspace_bytes(m, n, slices, "f16")
        assert nbytes == (2 * m * n * slices if slices > 1 else 0)
        ws = torch.full((nbytes // 2 + 8,), float("nan"), dtype=torch.float16, device="cuda") if nbytes else None
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm_splitk_serial(add, mult, to_device(A), to_device(B), to_device(C), dD, slices, ws, f(alpha), f(beta), f(ident), f(one), dtype="f16")
        torch.cuda.synchronize()
        assert_same_bits(dD.cpu().numpy(), want, f"serial split-K f16 {add}-{mult} {layouts} S={slices}")


# ---- the hand-scheduled 256 x 256 matrix-core tile (whole tiles of k-contiguous operands that fill the chip) ----

def test_hand_scheduled_matrix_core_tile(oracle, lib):
    """192 tiles and more of 256 x 256, A row-major and B column-major, kernel = mfma: exact on small integers
    (fragment layout, ring of stages, epilogue), one to nine stages of 32 k; then uniform data against a
    double-precision product within one binary16 rounding plus the error of a float sum."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m, n = 4096, 3072
    # (whole stages of 64 k take the form that fetches 128 bytes of k per row: one, two, three, ten stages of its ring of five)
    for k, (alpha, beta) in [(32, (1, 0)), (64, (1, 1)), (96, (2, -1)), (288, (-1, 2)), (128, (1, 1)), (192, (1, -1)), (640, (2, 1))]:
        A = inputs.integers(21 + k, m, k, -2, 2, np.float16, "C")
        B = inputs.integers(22 + k, k, n, -2, 2, np.float16, "F")
        C = inputs.integers(23 + k, m, n, -8, 8, np.float16, "C")
        want = oracle.srgemm("plus", "multiplies", A, B, C, np.float16(alpha), np.float16(beta), np.float16(0))
        assert np.abs(want.astype(np.float64)).max() <= 2048
        dD = to_device(np.full_like(C, 7))
        cuasr_amd.srgemm("plus", "multiplies", to_device(A), to_device(B), to_device(C), dD, np.float16(alpha), np.float16(beta),
                         np.float16(0), np.float16(1), dtype="f16", kernel="mfma")
        torch.cuda.synchronize()
        assert_same_bits(dD.cpu().numpy(), want, f"plus-times f16 mfma {m}x{n}x{k}")
    k = 1024
    A = inputs.uniform(31, m, k, -1.0, 1.0, np.float16, "C")
    B = inputs.uniform(32, k, n, -1.0, 1.0, np.float16, "F")
    C = inputs.uniform(33, m, n, -4.0, 4.0, np.float16, "C")
    alpha, beta = np.float16(0.75), np.float16(-1.5)
    r = float(alpha) * (A.astype(np.float64) @ B.astype(np.float64)) + float(beta) * C.astype(np.float64)
    bound = 2.0 ** -11 * np.abs(r) + 1e-5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + 1e-7
    dD = to_device(np.zeros_like(C))
    cuasr_amd.srgemm("plus", "multiplies", to_device(A), to_device(B), to_device(C), dD, alpha, beta, np.float16(0), np.float16(1),
                     dtype="f16", kernel="mfma")
    torch.cuda.synchronize()
    err = np.abs(dD.cpu().numpy().astype(np.float64) - r)
    assert (err <= bound).all(), f"worst excess {(err - bound).max():.3e}"


def test_hand_scheduled_matrix_core_tile_batch(oracle, lib):
    """13 products of 16 tiles of 256 x 256 each in one launch of the hand-scheduled tile (three stages of 32 k: the two-stage
    statement once and the single one), exact on small integers."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m = n = 1024
    batch = 13
    one, zero = np.float16(1), np.float16(0)
    for k in (96, 192):   # stages of 32 k; whole stages of 64 k (the form that fetches 128 bytes of k per row)
        A = inputs.integers(41 + k, batch * m, k, -2, 2, np.float16, "C").reshape(batch, m, k)
        B = inputs.integers(42 + k, batch * n, k, -2, 2, np.float16, "C").reshape(batch, n, k)        # column-major k x n slices
        C = inputs.integers(43 + k, batch * m, n, -8, 8, np.float16, "C").reshape(batch, m, n)
        dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda().transpose(1, 2), torch.from_numpy(C).cuda()
        dD = torch.zeros_like(dC)
        cuasr_amd.srgemm_batched("plus", "multiplies", dA, dB, dC, dD, one, one, zero, one, dtype="f16", kernel="mfma")
        torch.cuda.synchronize()
        got = dD.cpu().numpy()
        for i in (0, 5, 12):
            want = oracle.srgemm("plus", "multiplies", A[i], np.asfortranarray(B[i].T), C[i], one, one, zero)
            assert np.abs(want.astype(np.float64)).max() <= 2048
            assert_same_bits(got[i], want, f"batch product {i}, k = {k}")

