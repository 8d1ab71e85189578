"""Serial split-K (the reference's SplitKSerial = true, device/srgemm.h:218-282 and
kernel/srgemm.h:249-320) through the C ABI, against the oracle's model of the reference's
chain of epilogues.  Inputs are small integers wherever a sum is involved, so the result does
not depend on the order of additions inside a slice; where it depends on the slice boundaries
(alpha < 0 with a min/max over products) the library follows the reference's boundaries."""
import numpy as np
import pytest

from helpers import assert_same_bits, order_of, to_device, to_host

pytestmark = pytest.mark.gpu

NPD = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "u32": np.uint32}


def workspace(m, n, slices, dtype, poison=True):
    import torch
    import cuasr_amd
    nbytes = cuasr_amd.splitk_serial_workspace_bytes(m, n, slices, dtype)
    assert nbytes == (NPD[dtype]().itemsize * m * n * slices if slices > 1 else 0)
    if nbytes == 0:
        return None
    ws = torch.empty(nbytes // 4, dtype=torch.int32, device="cuda")
    if poison:
        ws.fill_(0x7FC00000)  # stale contents (a NaN pattern) must not reach the result
    return ws


def run(oracle, add, mult, dtype, m, n, k, layouts, kernel, alpha, beta, ident, one, slices, seed=21, lo=-8, hi=8, alias=False):
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    npd = NPD[dtype]
    if dtype == "u32":
        A = inputs.words32(seed, m, k, order_of(la))
        B = inputs.words32(seed + 1, k, n, order_of(lb))
        C = inputs.words32(seed + 2, m, n, order_of(lc))
    else:
        A = inputs.integers(seed, m, k, lo, hi, npd, order_of(la))
        B = inputs.integers(seed + 1, k, n, lo, hi, npd, order_of(lb))
        C = inputs.integers(seed + 2, m, n, lo, hi, npd, order_of(lc))
    want = oracle.srgemm_splitk_serial(add, mult, A, B, C, alpha, beta, ident, one, slices)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD = dC if alias else to_device(np.zeros_like(C))
    ws = workspace(m, n, slices, dtype)
    cuasr_amd.srgemm_splitk_serial(add, mult, dA, dB, dC, dD, slices, ws, alpha, beta, ident, one, dtype=dtype, kernel=kernel)
    torch.cuda.synchronize()
    assert_same_bits(to_host(dD, dtype), want, f"serial split-K {add}-{mult} {dtype} {m}x{n}x{k} {layouts} {kernel} S={slices}")


INF = float("inf")
FULL = 0xFFFFFFFF
# (add, mult, dtype, alpha, beta, add identity, mult identity)
CASES = {
    "minplus_beta_one": ("minimum", "plus", "f32", 3.0, 0.0, INF, 0.0),
    "minplus_beta_zero": ("minimum", "plus", "f32", 3.0, INF, INF, 0.0),
    "maxplus_f64": ("maximum", "plus", "f64", -1.0, 0.0, -INF, 0.0),
    "maxmin_f64": ("maximum", "minimum", "f64", 5.0, INF, -INF, INF),
    "plustimes_f32": ("plus", "multiplies", "f32", 2.0, -3.0, 0.0, 1.0),
    "plustimes_f64": ("plus", "multiplies", "f64", 2.0, -3.0, 0.0, 1.0),
    "mintimes_negative_alpha": ("minimum", "multiplies", "f32", -2.0, 1.0, INF, 1.0),
    "maxtimes_negative_alpha": ("maximum", "multiplies", "f64", -2.0, 1.0, -INF, 1.0),
    "xorand_u32": ("bit_xor", "bit_and", "u32", FULL, FULL, 0, FULL),
    "orand_i32": ("logical_or", "logical_and", "i32", 1, 1, 0, 1),
}


@pytest.mark.parametrize("slices", [1, 2, 3, 8, 40])
@pytest.mark.parametrize("case", sorted(CASES))
def test_serial_splitk_default_kernel(oracle, lib, case, slices):
    add, mult, dtype, alpha, beta, ident, one = CASES[case]
    lo, hi = (0, 2) if dtype == "i32" else (-8, 8)
    run(oracle, add, mult, dtype, 100, 60, 333, "ccc", "auto", alpha, beta, ident, one, slices, lo=lo, hi=hi)
    run(oracle, add, mult, dtype, 128, 132, 1000, "rcr", "auto", alpha, beta, ident, one, slices, lo=lo, hi=hi)


@pytest.mark.parametrize("kernel", ["naive", "valu", "direct", "mfma"])
@pytest.mark.parametrize("case", ["minplus_beta_one", "minplus_beta_zero", "maxplus_f64", "plustimes_f32", "plustimes_f64",
                                  "mintimes_negative_alpha", "xorand_u32"])
def test_serial_splitk_every_family(oracle, lib, case, kernel):
    import cuasr_amd
    add, mult, dtype, alpha, beta, ident, one = CASES[case]
    ran = 0
    for layouts, shape in (("rcr", (256, 128, 1040)), ("ccc", (260, 132, 520)), ("crr", (128, 256, 264))):
        for slices in (3, 8):
            try:
                run(oracle, add, mult, dtype, *shape, layouts, kernel, alpha, beta, ident, one, slices)
                ran += 1
            except cuasr_amd.CuasrError as e:
                assert e.status == 5, e  # kErrorNotSupported: this family does not run this semiring / element type
    if not ran:
        pytest.skip(f"{kernel} does not run {case}")


def test_serial_splitk_aliased_output_and_unread_source(oracle, lib):
    add, mult, dtype, alpha, beta, ident, one = CASES["minplus_beta_one"]
    run(oracle, add, mult, dtype, 130, 70, 500, "ccc", "auto", alpha, beta, ident, one, 4, alias=True)
    # beta = zero: C is not dereferenced (the reference's epilogue takes its no-source form), so NaNs there stay out
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m, n, k, slices = 96, 80, 400, 5
    A, B = inputs.integers(1, m, k, -8, 8, np.float32, "F"), inputs.integers(2, k, n, -8, 8, np.float32, "F")
    C = np.full((m, n), np.nan, dtype=np.float32, order="F")
    want = oracle.srgemm_splitk_serial("minimum", "plus", A, B, C, 3.0, INF, INF, 0.0, slices)
    assert not np.isnan(want).any()
    dD = to_device(np.zeros_like(C))
    cuasr_amd.srgemm_splitk_serial("minimum", "plus", to_device(A), to_device(B), to_device(C), dD, slices,
                                   workspace(m, n, slices, "f32"), 3.0, INF, INF, 0.0)
    torch.cuda.synchronize()
    assert_same_bits(to_host(dD, "f32"), want, "NaN source, beta = zero")


def test_serial_splitk_workspace_contract(lib):
    """A null workspace is an error only when there is more than one slice (device/srgemm.h:246-251)."""
    import torch
    import cuasr_amd
    A = torch.zeros(64, 64, device="cuda")
    D = torch.zeros(64, 64, device="cuda")
    with pytest.raises(cuasr_amd.CuasrError) as e:
        cuasr_amd.srgemm_splitk_serial("minimum", "plus", A, A, A, D, 2, None, 0.0, 0.0, INF, 0.0)
    assert e.value.status == 6  # kErrorWorkspaceNull
    cuasr_amd.srgemm_splitk_serial("minimum", "plus", A, A, A, D, 1, None, 0.0, 0.0, INF, 0.0)
    torch.cuda.synchronize()
    assert float(D.max()) == 0.0


def test_serial_splitk_deep_k_uniform_data(oracle, lib):
    """256 x 256 x 65536 min-plus on uniform [0, 10) data, the split-K example's shape: the chain of an
    idempotent, order-free add equals the unsplit product bit for bit (examples/02_splitk_srgemm/splitk_srgemm.cu:270-287)."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m = n = 256
    k = 65536
    A = inputs.uniform(31, m, k, 0, 10, order="C")
    B = inputs.uniform(32, k, n, 0, 10, order="F")
    C = inputs.uniform(33, m, n, 0, 10, order="C")
    want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, INF)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    for slices in (8, 16, 64):
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm_splitk_serial("minimum", "plus", dA, dB, dC, dD, slices, workspace(m, n, slices, "f32"),
                                       0.0, 0.0, INF, 0.0)
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, "f32"), want, f"S={slices}")


def test_serial_splitk_plus_times_tolerance(oracle, lib):
    """plus-times on N(0,1) data: |d - r| <= 1e-5 * sum_k |a||b| against the oracle's serial model."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m, n, k, slices = 256, 192, 4096, 6
    A, B, C = inputs.normal(41, m, k), inputs.normal(42, k, n), inputs.normal(43, m, n)
    want = oracle.srgemm_splitk_serial("plus", "multiplies", A, B, C, 1.5, -0.5, 0.0, 1.0, slices).astype(np.float64)
    dD = to_device(np.zeros_like(C))
    cuasr_amd.srgemm_splitk_serial("plus", "multiplies", to_device(A), to_device(B), to_device(C), dD, slices,
                                   workspace(m, n, slices, "f32"), 1.5, -0.5, 0.0, 1.0)
    torch.cuda.synchronize()
    got = to_host(dD, "f32").astype(np.float64)
    bound = 1e-5 * (1.5 * np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64) + 0.5 * np.abs(C))
    assert (np.abs(got - want) <= bound).all()


# ---- small outputs: several workgroups per slice --------------------------------------------------------------

SHARED = {
    "minplus_f32": ("minimum", "plus", "f32", 2.0, 0.0, INF, 0.0),
    "maxplus_f32_beta_zero": ("maximum", "plus", "f32", 0.0, -INF, -INF, 0.0),
    "maxmin_f32": ("maximum", "minimum", "f32", INF, INF, -INF, INF),
    "minplus_i32": ("minimum", "plus", "i32", 1, 0, 2**31 - 1, 0),
    "maxplus_u32": ("maximum", "plus", "u32", 0, 0, 0, 0),
    "xorand_u32": ("bit_xor", "bit_and", "u32", FULL, FULL, 0, FULL),
}


@pytest.mark.parametrize("form", ["parallel", "serial"])
@pytest.mark.parametrize("case", sorted(SHARED))
def test_splitk_of_a_small_output_shares_each_slice_between_workgroups(oracle, lib, case, form):
    """An output of few tiles in few slices (the shape of the 256 x 256 x 65536 split-K in 8 slices): the staged
    tiles give every slice's k range to several workgroups, which fold their parts into the slice's partial
    tile with native atomics after the workspace has been set to the additive identity.  Stale workspace
    contents, ragged extents, k that does not divide, and the serial form's chain (alpha multiplies every
    slice's partial) must all come out as the oracle's models say."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    add, mult, dtype, alpha, beta, ident, one = SHARED[case]
    for (m, n, k, slices, layouts) in [(256, 256, 16384, 8, "rcr"), (250, 130, 9001, 3, "ccc"), (64, 64, 40000, 2, "crc"), (100, 300, 6144, 4, "rrc")]:
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        npd = NPD[dtype]
        if dtype == "u32" and add == "bit_xor":
            A, B, C = inputs.words32(31, m, k, order_of(la)), inputs.words32(32, k, n, order_of(lb)), inputs.words32(33, m, n, order_of(lc))
        else:
            lo, hi = (0, 1000) if dtype == "u32" else (-1000, 1000)
            A = inputs.integers(31, m, k, lo, hi, npd, order_of(la))
            B = inputs.integers(32, k, n, lo, hi, npd, order_of(lb))
            C = inputs.integers(33, m, n, 2 * lo, 2 * hi, npd, order_of(lc))
        model = oracle.srgemm_splitk if form == "parallel" else oracle.srgemm_splitk_serial
        want = model(add, mult, A, B, C, alpha, beta, ident, one, slices, tbk=16 if form == "parallel" else 8)
        dA, dB, dC = to_device(A), to_device(B), to_device(C)
        dD = to_device(np.zeros_like(C))
        ws = torch.full((m * n * slices,), 0x7FC00000, dtype=torch.int32, device="cuda")   # stale contents must not survive
        run_it = cuasr_amd.srgemm_splitk if form == "parallel" else cuasr_amd.srgemm_splitk_serial
        run_it(add, mult, dA, dB, dC, dD, slices, ws, alpha, beta, ident, one, dtype=dtype)
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, dtype), want, f"{form} split-K {case} {m}x{n}x{k} {layouts} S={slices}")
