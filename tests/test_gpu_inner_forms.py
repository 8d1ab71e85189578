"""The two semirings whose staged-tile inner loop does not compute with the operators as written:
min-times / max-times (hardware min / max in the loop, the sign of a zero result restored
afterwards) and or-and on 4-byte types (panels staged as masks, one and-or per term).  Data here is
chosen so that the cases those forms must get right actually occur: zero results of both signs,
zero and non-zero operands of either sign."""
import numpy as np
import pytest

from helpers import assert_same_bits, order_of, to_device, to_host

pytestmark = pytest.mark.gpu

NPD = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "u32": np.uint32}
INF = float("inf")


def launch(add, mult, dtype, A, B, C, alpha, beta, ident, one, kernel, splitk=0, serial=False):
    import torch
    import cuasr_amd
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD = to_device(np.zeros_like(C))
    m, n = C.shape
    if splitk:
        ws = torch.empty(NPD[dtype]().itemsize * m * n * splitk // 4 + 4, dtype=torch.int32, device="cuda")
        fn = cuasr_amd.srgemm_splitk_serial if serial else cuasr_amd.srgemm_splitk
        fn(add, mult, dA, dB, dC, dD, splitk, ws, alpha, beta, ident, one, dtype=dtype, kernel=kernel)
    else:
        cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, alpha, beta, ident, one, dtype=dtype, kernel=kernel)
    torch.cuda.synchronize()
    return to_host(dD, dtype)


def signed_zero_counts(x):
    z = x[x == 0]
    return int(np.signbit(z).sum()), int((~np.signbit(z)).sum())


@pytest.mark.parametrize("kernel", ["auto", "valu", "naive"])
@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("add", ["minimum", "maximum"])
def test_times_semirings_zero_results_keep_the_reference_sign(oracle, lib, add, dtype, kernel):
    from cuasr_amd import inputs
    npd = NPD[dtype]
    ident = INF if add == "minimum" else -INF
    seen_neg = seen_pos = 0
    for layouts, (m, n, k) in (("ccc", (17, 27, 1)), ("rcr", (33, 20, 2)), ("crr", (64, 64, 5)), ("rrc", (130, 70, 37)),
                               ("ccc", (256, 256, 64)), ("rcr", (128, 132, 203))):
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        # one sign per operand, with zeros: every product is >= 0 (minimum) or <= 0 (maximum) and many are +0 or -0,
        # so the result is a zero wherever a zero product exists and its sign is that of the last one
        if add == "minimum":
            A = inputs.integers(1, m, k, -3, 0, npd, order_of(la))   # <= 0
            B = inputs.integers(2, k, n, -3, 0, npd, order_of(lb))   # <= 0
        else:
            A = inputs.integers(1, m, k, 0, 3, npd, order_of(la))    # >= 0
            B = inputs.integers(2, k, n, -3, 0, npd, order_of(lb))   # <= 0
        C = inputs.integers(3, m, n, -3, 3, npd, order_of(lc))
        for beta in (1.0, 0.0):
            want = oracle.srgemm(add, "multiplies", A, B, C, 1.0, beta, ident)
            neg, pos = signed_zero_counts(want)
            seen_neg += neg
            seen_pos += pos
            got = launch(add, "multiplies", dtype, A, B, C, 1.0, beta, ident, 1.0, kernel)
            assert_same_bits(got, want, f"{add}-times {dtype} {m}x{n}x{k} {layouts} {kernel} beta={beta}")
        # mixed signs as well (small integers, zero results are rarer)
        A = inputs.integers(4, m, k, -3, 3, npd, order_of(la))
        B = inputs.integers(5, k, n, -3, 3, npd, order_of(lb))
        want = oracle.srgemm(add, "multiplies", A, B, C, -2.0, 1.0, ident)
        got = launch(add, "multiplies", dtype, A, B, C, -2.0, 1.0, ident, 1.0, kernel)
        assert_same_bits(got, want, f"{add}-times {dtype} {m}x{n}x{k} {layouts} {kernel} mixed signs")
    assert seen_neg > 100 and seen_pos > 100, "the inputs must produce zero results of both signs"


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("add", ["minimum", "maximum"])
def test_times_semirings_split_k(oracle, lib, add, dtype):
    from cuasr_amd import inputs
    npd = NPD[dtype]
    ident = INF if add == "minimum" else -INF
    m, n, k = 96, 80, 333
    A = inputs.integers(1, m, k, -3, 0, npd, "C")
    B = inputs.integers(2, k, n, -3, 0, npd, "F") if add == "minimum" else inputs.integers(2, k, n, 0, 3, npd, "F")
    C = inputs.integers(3, m, n, -3, 3, npd, "C")
    for slices in (3, 8):
        want = oracle.srgemm_splitk(add, "multiplies", A, B, C, 1.0, 1.0, ident, 1.0, slices, tbk=16)
        got = launch(add, "multiplies", dtype, A, B, C, 1.0, 1.0, ident, 1.0, "valu", splitk=slices)
        # the parallel form folds the slices' zeros with add(acc, partial): which zero survives depends on where the
        # slices end, and this library's slices differ from the reference's -- the value is the same, the sign may not be
        assert np.array_equal(got, want)
        want = oracle.srgemm_splitk_serial(add, "multiplies", A, B, C, 1.0, 1.0, ident, 1.0, slices)
        got = launch(add, "multiplies", dtype, A, B, C, 1.0, 1.0, ident, 1.0, "valu", splitk=slices, serial=True)
        assert_same_bits(got, want, f"serial split-K {add}-times {dtype} S={slices}")


def sparse(seed, rows, cols, npd, order, density=0.08):
    """Mostly zeros; the rest of either sign (floating point) or any non-zero value (integers)."""
    from cuasr_amd import inputs
    mask = inputs.bernoulli(seed, rows, cols, density, np.int32, order)
    if npd in (np.float32, np.float64):
        vals = inputs.uniform(seed + 100, rows, cols, -2.0, 2.0, npd, order)
    else:
        vals = inputs.integers(seed + 100, rows, cols, 1, 1000, npd, order)
    return (mask.astype(npd) * vals).astype(npd, order=order)


@pytest.mark.parametrize("kernel", ["auto", "valu", "direct", "naive"])
@pytest.mark.parametrize("dtype", ["f32", "i32", "u32", "f64"])
def test_or_and_on_truth_values_of_arbitrary_operands(oracle, lib, dtype, kernel):
    """binary_and / binary_or (functional.h:212, :252) see only whether an operand is zero; the result is 1 or 0."""
    import cuasr_amd
    npd = NPD[dtype]
    ones = zeros = ran = 0
    for layouts, (m, n, k) in (("ccc", (17, 27, 1)), ("rcr", (33, 20, 23)), ("crr", (64, 64, 64)), ("rrc", (130, 70, 37)),
                               ("ccc", (256, 384, 100)), ("rcr", (128, 132, 520))):
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        A, B = sparse(11, m, k, npd, order_of(la)), sparse(12, k, n, npd, order_of(lb))
        C = sparse(13, m, n, npd, order_of(lc), 0.3)
        if dtype in ("f32", "f64"):
            A.flat[::17], B.flat[::19], C.flat[::23] = npd("nan"), npd("-inf"), npd("nan")   # true, all of them
            A.flat[1::17] = npd(-0.0)                                                        # false
        for alpha, beta in ((1, 0), (1, 1), (0, 1), (7, 3)):   # any non-zero scalar is "true"
            want = oracle.srgemm("logical_or", "logical_and", A, B, C, alpha, beta, 0)
            try:
                got = launch("logical_or", "logical_and", dtype, A, B, C, alpha, beta, 0, 1, kernel)
            except cuasr_amd.CuasrError as e:
                assert e.status == 5 and kernel == "direct", e   # shapes the direct tile does not take
                continue
            assert_same_bits(got, want, f"or-and {dtype} {m}x{n}x{k} {layouts} {kernel} alpha={alpha} beta={beta}")
            ran += 1
            if (alpha, beta) == (1, 0):
                ones += int((want == 1).sum())
                zeros += int((want == 0).sum())
    if not ran:
        pytest.skip(f"{kernel} does not run or-and on {dtype}")
    assert ones > 1000 and zeros > 1000, "the inputs must produce both truth values"


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u32"])
@pytest.mark.parametrize("layouts", ["ccc", "rcr", "crr", "rrc", "rrr", "ccr"])
def test_or_and_large_outputs_on_packed_masks(oracle, lib, dtype, layouts):
    """From 384 tiles of 128 x 256 on (double: 128), or-and on 4- and 8-byte operands runs on the 16-bit mask tile: whole tiles of
    aligned operands, ragged extents, an identity that is not zero, scalars that are zero, and floating-point operands
    that hold -0 (false), NaN and infinities (true, functional.h:212)."""
    import cuasr_amd
    npd = NPD[dtype]
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for (m, n, k), ident, alpha, beta in (((4096, 3072, 64), 0, 1, 1), ((4000, 4100, 37), 0, 1, 0), ((4000, 4100, 37), 0, 0, 1),
                                          ((3968, 3328, 33), 2.5, 1, 1), ((2048, 2048, 40), 0, 1, 0)):   # (the last: on masks for f64 only)
        A, B = sparse(31, m, k, npd, order_of(la), 0.06), sparse(32, k, n, npd, order_of(lb), 0.06)
        C = sparse(33, m, n, npd, order_of(lc), 0.3)
        if dtype in ("f32", "f64"):
            A[::7, ::3] = npd(-0.0)
            A[5::11, 1::4] = npd("nan")
            B[2::13, ::5] = npd("inf")
        ident = ident if dtype in ("f32", "f64") else int(ident)
        want = oracle.srgemm("logical_or", "logical_and", A, B, C, alpha, beta, ident)
        print(f"or-and {dtype} {m}x{n}x{k} {layouts} ident={ident} alpha={alpha} beta={beta}", flush=True)
        for kernel in ("auto", "valu"):
            got = launch("logical_or", "logical_and", dtype, A, B, C, alpha, beta, ident, 1, kernel)
            assert_same_bits(got, want, f"or-and {dtype} {m}x{n}x{k} {layouts} {kernel} ident={ident} alpha={alpha} beta={beta}")
        if ident == 0 and (alpha, beta) == (1, 0):
            assert 0.05 < (want == 1).mean() < 0.95, "the inputs must produce both truth values"
    dA = to_device(np.zeros((4096, 64), npd))
    dB = to_device(np.zeros((64, 3072), npd))
    dD = to_device(np.zeros((4096, 3072), npd))
    assert lib.cuasr_amd_selected_kernel(cuasr_amd.make_desc("logical_or", "logical_and", dtype, dA, dB, dD, dD, 1, 1, 0, 1)) == b"valu"


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32"])
def test_or_and_split_k_on_packed_masks(oracle, lib, dtype):
    """Slices count towards the 384 workgroups: 8 x 8 tiles in 6 or 7 slices run the mask tile into the workspace."""
    npd = NPD[dtype]
    m, n, k = 1024, 2048, 700
    A, B, C = sparse(41, m, k, npd, "C", 0.02), sparse(42, k, n, npd, "F", 0.02), sparse(43, m, n, npd, "C", 0.3)
    for slices in (6, 7):
        for beta in (0, 1):
            want = oracle.srgemm("logical_or", "logical_and", A, B, C, 1, beta, 0)
            got = launch("logical_or", "logical_and", dtype, A, B, C, 1, beta, 0, 1, "valu", splitk=slices)
            assert_same_bits(got, want, f"split-K or-and {dtype} S={slices} beta={beta}")
            got = launch("logical_or", "logical_and", dtype, A, B, C, 1, beta, 0, 1, "valu", splitk=slices, serial=True)
            assert_same_bits(got, want, f"serial split-K or-and {dtype} S={slices} beta={beta}")


@pytest.mark.parametrize("dtype", ["f32", "i32"])
def test_or_and_split_k(oracle, lib, dtype):
    npd = NPD[dtype]
    m, n, k = 96, 80, 1000
    A, B, C = sparse(21, m, k, npd, "C", 0.02), sparse(22, k, n, npd, "F", 0.02), sparse(23, m, n, npd, "C", 0.3)
    for slices in (3, 8, 70):
        for beta in (0, 1):
            want = oracle.srgemm("logical_or", "logical_and", A, B, C, 1, beta, 0)
            got = launch("logical_or", "logical_and", dtype, A, B, C, 1, beta, 0, 1, "valu", splitk=slices)
            assert_same_bits(got, want, f"split-K or-and {dtype} S={slices} beta={beta}")
            got = launch("logical_or", "logical_and", dtype, A, B, C, 1, beta, 0, 1, "valu", splitk=slices, serial=True)
            assert_same_bits(got, want, f"serial split-K or-and {dtype} S={slices} beta={beta}")
