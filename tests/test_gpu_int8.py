"""int8 operands with int32 accumulation (the element types of the reference's dp4a cores) against the CPU
oracle, bit for bit, through the C ABI: plus-times on the matrix cores in every layout, aligned and ragged,
the other operator pairs on the naive kernel, split-K, batches."""
import numpy as np
import pytest

from helpers import assert_same_bits, order_of, to_device

pytestmark = pytest.mark.gpu

LAYOUTS = ["ccc", "rrr", "crc", "rcr", "rcc", "crr", "ccr", "rrc"]


def operands(m, n, k, la, lb, lc, seed=1):
    from cuasr_amd import inputs
    A = inputs.integers(seed, m, k, -128, 127, np.int8, order_of(la))
    B = inputs.integers(seed + 1, k, n, -128, 127, np.int8, order_of(lb))
    C = inputs.integers(seed + 2, m, n, -100000, 100000, np.int32, order_of(lc))
    return A, B, C


def check(oracle, add, mult, m, n, k, layouts, kernel="auto", alpha=None, beta=None, splitk=0, seed=1):
    import torch
    import cuasr_amd
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    A, B, C = operands(m, n, k, la, lb, lc, seed)
    ident = int(cuasr_amd.op_identity(add, "i8"))
    one = int(cuasr_amd.op_identity(mult, "i8"))
    alpha = one if alpha is None else alpha
    beta = one if beta is None else beta
    want = oracle.srgemm(add, mult, A, B, C, alpha, beta, ident)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD = to_device(np.zeros_like(C))
    print(f"int8 {add}-{mult} {m}x{n}x{k} {layouts} {kernel} alpha={alpha} beta={beta} splitk={splitk}", flush=True)
    if splitk:
        ws = torch.empty(cuasr_amd.splitk_workspace_bytes(m, n, splitk, "i8") // 4 + 4, dtype=torch.int32, device="cuda")
        cuasr_amd.srgemm_splitk(add, mult, dA, dB, dC, dD, splitk, ws, alpha, beta, ident, one, dtype="i8", kernel=kernel)
    else:
        cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, alpha, beta, ident, one, dtype="i8", kernel=kernel)
    torch.cuda.synchronize()
    assert_same_bits(dD.cpu().numpy(), want, f"{add}-{mult} i8 {m}x{n}x{k} {layouts} {kernel}")


@pytest.mark.parametrize("layouts", LAYOUTS)
def test_plus_times_on_the_matrix_cores(oracle, lib, layouts):
    # whole tiles of aligned operands (the unguarded kernel), then ragged / tiny / thin ones (the guarded one)
    for shape in [(128, 128, 64), (256, 384, 192), (100, 70, 45), (1, 1, 1), (130, 258, 67), (64, 8, 200), (16, 16, 16)]:
        check(oracle, "plus", "multiplies", *shape, layouts, "mfma")
        check(oracle, "plus", "multiplies", *shape, layouts, "auto", alpha=3, beta=-2)
        check(oracle, "plus", "multiplies", *shape, layouts, "auto", alpha=1, beta=0)


def test_selected_family(lib):
    import cuasr_amd
    dA = to_device(np.zeros((128, 64), np.int8))
    dB = to_device(np.zeros((64, 256), np.int8))
    dD = to_device(np.zeros((128, 256), np.int32))
    for (add, mult), name in [(("plus", "multiplies"), b"mfma"), (("minimum", "plus"), b"valu"), (("maximum", "minimum"), b"valu"),
                              (("logical_or", "logical_and"), b"valu"), (("bit_xor", "bit_and"), b"valu"), (("bit_or", "bit_and"), b"valu"),
                              (("bit_xor", "logical_and"), b"naive"), (("minimum", "multiplies"), b"valu"),
                              (("maximum", "multiplies"), b"valu")]:
        desc = cuasr_amd.make_desc(add, mult, "i8", dA, dB, dD, dD, 1, 0, 0, 1)
        assert lib.cuasr_amd_selected_kernel(desc) == name


@pytest.mark.parametrize("sr", [("minimum", "plus"), ("maximum", "plus"), ("minimum", "maximum"), ("maximum", "minimum"),
                                ("logical_or", "logical_and"), ("bit_xor", "bit_and"), ("bit_or", "bit_and"),
                                ("minimum", "multiplies"), ("plus", "multiplies")])
def test_every_pair_on_widened_operands(oracle, lib, sr):
    for layouts in ("ccc", "rcr"):
        check(oracle, *sr, 70, 90, 33, layouts, "auto")
        check(oracle, *sr, 70, 90, 33, layouts, "naive")


@pytest.mark.parametrize("sr", [("minimum", "plus"), ("maximum", "plus"), ("minimum", "maximum"), ("maximum", "minimum"),
                                ("minimum", "multiplies"), ("maximum", "multiplies"), ("bit_xor", "bit_and"), ("bit_or", "bit_and")])
@pytest.mark.parametrize("layouts", LAYOUTS)
def test_tropical_pairs_on_the_packed_tile(oracle, lib, sr, layouts):
    """Sums, minima and maxima of two int8 values are exact in binary16: these pairs run on the packed
    half-precision tile (operands converted on their way to LDS, integer epilogue); products of two int8 values are
    exact as 16-bit integers: min-times and max-times run on the same tile with int16 lanes, and so do the bitwise
    pairs (and / xor / or of sign-extended bytes are the sign extensions of the byte results).  Every tile size,
    aligned and ragged, identities and scalars that are not the semiring's own."""
    check(oracle, *sr, 100, 300, 45, layouts, "valu")                        # 16 x 128 tiles, k shared out between the waves, ragged
    check(oracle, *sr, 1530, 1300, 77, layouts, "valu", alpha=3, beta=-2)    # 32 x 128 tiles, likewise
    check(oracle, *sr, 520, 390, 9, layouts, "valu")                         # k shorter than a tile
    check(oracle, *sr, 1, 1, 1, layouts, "valu")
    check(oracle, *sr, 2048, 2048, 96, layouts, "valu", alpha=7, beta=-3)    # 64 x 128 tiles
    check(oracle, *sr, 4096, 4096, 64, layouts, "valu")                      # full tiles, unguarded
    check(oracle, *sr, 4000, 4100, 70, layouts, "valu", alpha=-100, beta=100)  # full tiles, guarded


@pytest.mark.parametrize("layouts", ["ccc", "rcr", "crr", "rrc"])
def test_boolean_closure_on_masks(oracle, lib, layouts):
    """or-and on int8 operands: sparse (most entries zero), so that the answer is not all ones; every tile size;
    an identity that is not zero."""
    import torch
    import cuasr_amd
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    rng = np.random.default_rng(23)
    for (m, n, k), ident in [((1024, 1024, 64), 0), ((2048, 2048, 40), 0), ((4096, 4096, 32), 0), ((4000, 4100, 37), 0),
                             ((300, 200, 45), 7), ((70, 90, 1), 0), ((1530, 1300, 50), 0)]:
        A = np.asarray(np.where(rng.random((m, k)) < 0.03, rng.integers(-128, 128, (m, k)), 0).astype(np.int8), order=order_of(la))
        B = np.asarray(np.where(rng.random((k, n)) < 0.03, rng.integers(-128, 128, (k, n)), 0).astype(np.int8), order=order_of(lb))
        C = np.asarray(np.where(rng.random((m, n)) < 0.1, rng.integers(-5, 6, (m, n)), 0).astype(np.int32), order=order_of(lc))
        want = oracle.srgemm("logical_or", "logical_and", A, B, C, 1, 1, ident)
        assert ident != 0 or 0.02 < (want != 0).mean() < 0.98
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm("logical_or", "logical_and", to_device(A), to_device(B), to_device(C), dD, 1, 1, ident, 1, dtype="i8", kernel="valu")
        torch.cuda.synchronize()
        assert_same_bits(dD.cpu().numpy(), want, f"or-and i8 {m}x{n}x{k} {layouts} identity {ident}")


def test_products_at_the_ends_of_the_int16_range(oracle, lib):
    """min-times / max-times: (-128) (-128) = 16384 is the largest product, (-128) 127 = -16256 the smallest; rows and
    columns that hold nothing else, identities inside and outside the int16 range."""
    import torch
    import cuasr_amd
    rng = np.random.default_rng(5)
    for add in ("minimum", "maximum"):
        for (m, n, k), ident in [((130, 260, 40), 2 ** 31 - 1), ((130, 260, 40), 100), ((64, 128, 3), -40000), ((520, 390, 77), -(2 ** 31)),
                                 ((70, 90, 1), 12345)]:
            A = np.asarray(rng.choice(np.array([-128, 127, -1, 1], np.int8), (m, k)), order="C")
            B = np.asarray(rng.choice(np.array([-128, 127, -1, 1], np.int8), (k, n)), order="F")
            if k:
                A[::3, :] = -128
                B[:, ::5] = -128       # (rows x columns of nothing but 16384)
                B[:, 1::5] = 127
            C = np.asarray(rng.integers(-50000, 50000, (m, n)).astype(np.int32), order="C")
            want = oracle.srgemm(add, "multiplies", A, B, C, 1, 0, ident)
            dD = to_device(np.zeros_like(C))
            cuasr_amd.srgemm(add, "multiplies", to_device(A), to_device(B), to_device(C), dD, 1, 0, ident, 1, dtype="i8", kernel="valu")
            torch.cuda.synchronize()
            assert_same_bits(dD.cpu().numpy(), want, f"{add}-times i8 {m}x{n}x{k} identity {ident}")


def test_tropical_identity_that_is_not_infinite(oracle, lib):
    """The caller's additive identity takes part in the result (here it beats some of the sums), also with no
    terms at all."""
    import torch
    import cuasr_amd
    for (m, n, k) in [(70, 90, 33), (70, 90, 0)]:
        A, B, C = operands(m, n, k, "col", "row", "col", seed=5)
        C[:] = 1000                                                   # (out of the way: D = min(acc, 0 + C))
        want = oracle.srgemm("minimum", "plus", A, B, C, 0, 0, -225)
        dA, dB, dC = to_device(A), to_device(B), to_device(C)
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm("minimum", "plus", dA, dB, dC, dD, 0, 0, -225, 0, dtype="i8", kernel="valu")
        torch.cuda.synchronize()
        assert_same_bits(dD.cpu().numpy(), want, f"identity -225, k = {k}")
        assert k == 0 or (want == -225).any() and (want < -225).any()


@pytest.mark.parametrize("slices", [1, 3, 8])
def test_splitk(oracle, lib, slices):
    # sums of int32 wrap modulo 2^32 in any order: split-K is bit-exact for plus-times too
    for shape, layouts in [((256, 256, 1024), "ccc"), ((100, 60, 1000), "rcr"), ((128, 128, 192), "crc")]:
        check(oracle, "plus", "multiplies", *shape, layouts, "auto", alpha=2, beta=5, splitk=slices)
    check(oracle, "minimum", "plus", 100, 60, 1000, "ccc", "auto", splitk=slices)


def test_1024(oracle, lib):
    for layouts in ("ccc", "rcr", "crr"):
        check(oracle, "plus", "multiplies", 1024, 1024, 1024, layouts, "auto", alpha=1, beta=1)


@pytest.mark.parametrize("layouts", LAYOUTS)
def test_many_tiles(oracle, lib, layouts):
    """Hundreds of tiles and several k-tiles (the prefetch runs two tiles ahead): whole tiles of aligned operands,
    and ragged edges with an odd k (the guarded form)."""
    check(oracle, "plus", "multiplies", 3584, 3840, 640, layouts, "auto", alpha=1, beta=1)
    check(oracle, "plus", "multiplies", 3587, 3830, 333, layouts, "auto", alpha=-3, beta=2)


def test_wraparound(oracle, lib):
    """All operands at -128 and a long k: the int32 sums wrap, the same way on both sides."""
    import torch
    import cuasr_amd
    m, n, k = 128, 128, 200000
    A = np.full((m, k), -128, np.int8)
    B = np.full((k, n), -128, np.int8, order="F")
    C = np.zeros((m, n), np.int32)
    want = np.full((m, n), (16384 * k + 2 ** 31) % 2 ** 32 - 2 ** 31, np.int64).astype(np.int32)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD = to_device(np.zeros_like(C))
    cuasr_amd.srgemm("plus", "multiplies", dA, dB, dC, dD, 1, 0, 0, 1, dtype="i8")
    torch.cuda.synchronize()
    assert_same_bits(dD.cpu().numpy(), want, "wrapped sums")


def test_batch_in_the_grid(oracle, lib):
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    for (m, n, k, batch) in [(64, 64, 64, 9), (128, 128, 128, 3), (50, 30, 70, 4)]:
        A = inputs.integers(3, batch * m, k, -128, 127, np.int8, "C").reshape(batch, m, k)
        B = inputs.integers(4, batch * k, n, -128, 127, np.int8, "C").reshape(batch, k, n)
        C = inputs.integers(5, batch * m, n, -1000, 1000, np.int32, "C").reshape(batch, m, n)
        dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
        dD = torch.zeros_like(dC)
        cuasr_amd.srgemm_batched("plus", "multiplies", dA, dB, dC, dD, 1, 1, 0, 1, dtype="i8")
        torch.cuda.synchronize()
        got = dD.cpu().numpy()
        for i in range(batch):
            want = oracle.srgemm("plus", "multiplies", A[i], B[i], C[i], 1, 1, 0)
            assert_same_bits(got[i], want, f"batch product {i} of {m}x{n}x{k}")


@pytest.mark.parametrize("slices", [1, 2, 5])
def test_serial_splitk(oracle, lib, slices):
    """The serial split-K chain of epilogues on int8 operands (integer arithmetic: exact in any order)."""
    import torch
    import cuasr_amd
    for (add, mult, alpha, beta, ident, one), layouts in [(("plus", "multiplies", 2, -3, 0, 1), "rcr"),
                                                           (("minimum", "plus", 3, 0, 2 ** 31 - 1, 0), "ccc")]:
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        m, n, k = 130, 258, 200
        A, B, C = operands(m, n, k, la, lb, lc, seed=41)
        want = oracle.srgemm_splitk_serial(add, mult, A, B, C, alpha, beta, ident, one, slices)
        nbytes = cuasr_amd.splitk_serial_workspace_bytes(m, n, slices, "i8")
        assert nbytes == (4 * m * n * slices if slices > 1 else 0)
        ws = torch.full((nbytes // 4 + 4,), 0x7FC00000, dtype=torch.int32, device="cuda") if nbytes else None
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm_splitk_serial(add, mult, to_device(A), to_device(B), to_device(C), dD, slices, ws, alpha, beta, ident, one, dtype="i8")
        torch.cuda.synchronize()
        assert_same_bits(dD.cpu().numpy(), want, f"serial split-K i8 {add}-{mult} {layouts} S={slices}")


# ---- the hand-scheduled 256 x 256 tile (whole tiles of k-contiguous operands that fill the chip) ----------------

def test_hand_scheduled_tile_plain(oracle, lib):
    """192 tiles and more of 256 x 256 with A row-major and B column-major (both k-contiguous) take the
    hand-scheduled tile: one, two, three (the ring's prologue) and nine stages of 64 k, scalars that are not the
    semiring's own, and the same shape with one operand the other way round (the compiled kernel) for contrast."""
    # (whole stages of 128 k take the form that fetches 128 bytes of k per row: one, two, three, ten stages of its ring of five)
    for k in (64, 128, 192, 576, 256, 384, 1280):
        check(oracle, "plus", "multiplies", 4096, 3072, k, "rcr", "auto", alpha=3, beta=-2, seed=k)
    check(oracle, "plus", "multiplies", 3072, 4096, 320, "rcc", "mfma", alpha=1, beta=0)   # column-major C: the transposed problem
    check(oracle, "plus", "multiplies", 4096, 3072, 128, "ccr", "auto", alpha=1, beta=1)


def test_hand_scheduled_tile_splitk_and_batch(oracle, lib):
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    # 16 tiles x 13 slices of 64 k: every slice one stage; then slices of five stages with a ragged last slice
    check(oracle, "plus", "multiplies", 1024, 1024, 64 * 13, "rcr", "auto", alpha=2, beta=5, splitk=13)
    check(oracle, "plus", "multiplies", 1024, 1024, 64 * 61, "rcr", "auto", alpha=1, beta=1, splitk=13)
    # 13 products of 16 tiles each in one launch
    m = n = 1024
    batch = 13
    for k in (192, 384):   # stages of 64 k; whole stages of 128 k (the form that fetches 128 bytes of k per row)
        A = inputs.integers(3 + k, batch * m, k, -128, 127, np.int8, "C").reshape(batch, m, k)
        B = inputs.integers(4 + k, batch * n, k, -128, 127, np.int8, "C").reshape(batch, n, k)        # column-major k x n slices
        C = inputs.integers(5 + k, batch * m, n, -1000, 1000, np.int32, "C").reshape(batch, m, n)
        dA, dB, dC = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda().transpose(1, 2), torch.from_numpy(C).cuda()
        dD = torch.zeros_like(dC)
        cuasr_amd.srgemm_batched("plus", "multiplies", dA, dB, dC, dD, 1, 1, 0, 1, dtype="i8")
        torch.cuda.synchronize()
        got = dD.cpu().numpy()
        for i in (0, 5, 12):
            want = oracle.srgemm("plus", "multiplies", A[i], np.asfortranarray(B[i].T), C[i], 1, 1, 0)
            assert_same_bits(got[i], want, f"batch product {i}, k = {k}")
