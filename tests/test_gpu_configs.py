"""The five benchmark workloads at their full sizes, through the C ABI, against
the CPU oracle (bit-exact, or within the stated tolerance for plus-times)."""
import numpy as np
import pytest

from helpers import assert_same_bits, to_device, to_host

pytestmark = pytest.mark.gpu


def _run(add, mult, A, B, C, alpha, beta, ident, one, dtype, kernel="auto"):
    import torch
    import cuasr_amd
    dD = to_device(np.zeros_like(C))
    cuasr_amd.srgemm(add, mult, to_device(A), to_device(B), to_device(C), dD, alpha, beta, ident, one, dtype=dtype, kernel=kernel)
    torch.cuda.synchronize()
    return to_host(dD, dtype)


def test_config1_minplus_1024(oracle, lib):
    """min-plus f32, column-major, 1024^3, U[0,1), C = identity, alpha = one, beta = zero (and one)."""
    from cuasr_amd import inputs
    n = 1024
    A, B = inputs.uniform(101, n, n), inputs.uniform(102, n, n)
    for ident in (np.float32(np.inf), np.finfo(np.float32).max):  # +inf and the reference's numeric_limits::max
        C = np.full((n, n), ident, dtype=np.float32, order="F")
        want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, ident, ident)
        for kernel in ("auto", "mfma", "naive"):
            assert_same_bits(_run("minimum", "plus", A, B, C, 0.0, ident, ident, 0.0, "f32", kernel), want, kernel)
    C = inputs.uniform(103, n, n)
    want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf)
    assert_same_bits(_run("minimum", "plus", A, B, C, 0.0, 0.0, np.inf, 0.0, "f32"), want, "beta = one")


def test_config2_apsp_4096(oracle, lib):
    """APSP by repeated squaring: 12 steps of D <- min(D, D (x) D) at 4096, final matrix bit-exact;
    an integer-weight variant must equal Floyd-Warshall."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    n = 4096
    D0 = inputs.graph_distances(2024, n)
    host = D0
    for _ in range(12):
        host = oracle.srgemm("minimum", "plus", host, host, host, 0.0, 0.0, np.inf)
    cur = to_device(D0)
    bufs = [to_device(np.zeros_like(D0)) for _ in range(2)]
    for i in range(12):
        cuasr_amd.srgemm("minimum", "plus", cur, cur, cur, bufs[i & 1], 0.0, 0.0, float("inf"), 0.0)
        cur = bufs[i & 1]
    torch.cuda.synchronize()
    got = to_host(cur, "f32")
    assert_same_bits(got, host, "APSP 12 squarings")
    # closure properties that do not need the oracle: idempotent, zero diagonal, triangle inequality on a sample
    cuasr_amd.srgemm("minimum", "plus", cur, cur, cur, bufs[0] if cur is bufs[1] else bufs[1], 0.0, 0.0, float("inf"), 0.0)
    torch.cuda.synchronize()
    again = to_host(bufs[0] if cur is bufs[1] else bufs[1], "f32")
    assert_same_bits(again, got, "closed matrix is a fixed point")
    assert np.all(np.diag(got) == 0)
    # integer weights: every path length is exact in fp32, so the closure IS Floyd-Warshall's
    m = 256
    Di = inputs.graph_distances(7, m, density=0.05, integer_weights=True)
    cur = to_device(Di)
    b2 = [to_device(np.zeros_like(Di)) for _ in range(2)]
    for i in range(8):
        cuasr_amd.srgemm("minimum", "plus", cur, cur, cur, b2[i & 1], 0.0, 0.0, float("inf"), 0.0)
        cur = b2[i & 1]
    torch.cuda.synchronize()
    fw = Di.astype(np.float64).copy()
    for kk in range(m):
        fw = np.minimum(fw, fw[:, kk:kk + 1] + fw[kk:kk + 1, :])
    assert np.array_equal(to_host(cur, "f32").astype(np.float64), fw)


@pytest.mark.parametrize("ident", [-np.inf, np.finfo(np.float64).tiny], ids=["minus_inf", "reference_constant"])
@pytest.mark.parametrize("sr", ["max-plus", "max-min"])
def test_config3_f64_8192(oracle, lib, sr, ident):
    """fp64 max-plus / max-min at 8192^3, beta = one with a seeded C: a 512 x 512 block against the
    oracle bit-exact, the full matrix against the naive on-device kernel by checksum; with the
    accumulator starting from -inf and from the reference's own identity constant."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    n = 8192
    A = inputs.uniform(301, n, n, -1.0, 1.0, np.float64)
    B = inputs.uniform(302, n, n, -1.0, 1.0, np.float64)
    C = inputs.uniform(303, n, n, -1.0, 1.0, np.float64)
    add, mult = ("maximum", "plus") if sr == "max-plus" else ("maximum", "minimum")
    one = 0.0 if sr == "max-plus" else np.inf
    # additive identity: -inf, or the reference's maximum<double>::Identity = numeric_limits<double>::min()
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD, dN = to_device(np.zeros_like(C)), to_device(np.zeros_like(C))
    cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, one, one, ident, one, dtype="f64")
    cuasr_amd.srgemm(add, mult, dA, dB, dC, dN, one, one, ident, one, dtype="f64", kernel="naive")
    torch.cuda.synchronize()
    # full-matrix checksum of bit patterns, tuned kernel vs naive kernel
    x = dD.t().contiguous().view(torch.int64)
    y = dN.t().contiguous().view(torch.int64)
    assert int(x.sum()) == int(y.sum()) and bool(torch.equal(x, y))
    r0, c0 = 3 * 512 + 17, 9 * 512 + 5  # block position (not tile aligned)
    want = oracle.srgemm(add, mult, np.asfortranarray(A[r0:r0 + 512, :]), np.asfortranarray(B[:, c0:c0 + 512]),
                         np.asfortranarray(C[r0:r0 + 512, c0:c0 + 512]), one, one, ident)
    got = dD[r0:r0 + 512, c0:c0 + 512].cpu().numpy()
    assert_same_bits(np.asfortranarray(got), want, sr)


@pytest.mark.parametrize("layouts", ["tn", "nn"])
def test_config4_splitk(oracle, lib, layouts):
    """Split-K min-plus, M = N = 256, K = 65536, slices in {8, 16, 32, 64}; bit-exact vs oracle and vs non-split."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m = n = 256
    k = 65536
    oa, ob, oc = ("C", "F", "C") if layouts == "tn" else ("F", "F", "F")  # tn_t: K contiguous in A and B
    A = inputs.uniform(401, m, k, 0.0, 10.0, order=oa)
    B = inputs.uniform(402, k, n, 0.0, 10.0, order=ob)
    C = inputs.uniform(403, m, n, 0.0, 10.0, order=oc)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    inf = float("inf")
    for beta in (inf, 0.0):
        want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, beta, np.inf)
        plain = to_device(np.zeros_like(C))
        cuasr_amd.srgemm("minimum", "plus", dA, dB, dC, plain, 0.0, beta, inf, 0.0)
        torch.cuda.synchronize()
        assert_same_bits(to_host(plain, "f32"), want, "non-split")
        for slices in (8, 16, 32, 64):
            ws = torch.empty(cuasr_amd.splitk_workspace_bytes(m, n, slices, "f32") // 4, dtype=torch.float32, device="cuda")
            dD = to_device(np.zeros_like(C))
            cuasr_amd.srgemm_splitk("minimum", "plus", dA, dB, dC, dD, slices, ws, 0.0, beta, inf, 0.0)
            torch.cuda.synchronize()
            assert_same_bits(to_host(dD, "f32"), want, f"split-K S={slices} beta={beta}")


def test_config5a_xor_and_u32_4096(oracle, lib):
    """GF(2) product on bit-packed uint32 words, 4096^3: bitwise and with xor, bit-exact; plus the
    reference example's variant (logical and on 0/1 ints, 512^3)."""
    from cuasr_amd import inputs
    n = 4096
    A, B = inputs.words32(501, n, n), inputs.words32(502, n, n)
    C = np.zeros((n, n), dtype=np.uint32, order="F")
    want = oracle.srgemm("bit_xor", "bit_and", A, B, C, 0xFFFFFFFF, 0, 0)
    got = _run("bit_xor", "bit_and", A, B, C, 0xFFFFFFFF, 0, 0, 0xFFFFFFFF, "u32")
    assert_same_bits(got, want, "xor-and u32")
    # bit-plane spot check against an integer matmul mod 2 (independent of the oracle)
    rows = slice(100, 164)
    pa = ((A[rows, :] >> np.uint32(5)) & 1).astype(np.float64)
    pb = ((B[:, :256] >> np.uint32(5)) & 1).astype(np.float64)
    assert np.array_equal((got[rows, :256] >> np.uint32(5)) & 1, ((pa @ pb) % 2).astype(np.uint32))
    m = 512
    Ai, Bi, Ci = inputs.bernoulli(3090, m, m, 0.025), inputs.bernoulli(3091, m, m, 0.025), inputs.bernoulli(3092, m, m, 0.025)
    for beta in (0, 1):
        want = oracle.srgemm("bit_xor", "logical_and", Ai, Bi, Ci, 1, beta, 0)
        assert_same_bits(_run("bit_xor", "logical_and", Ai, Bi, Ci, 1, beta, 0, 1, "i32"), want, "example 01")


def test_config5b_plus_times_f32_4096(oracle, lib):
    """plus-times f32 control semiring, N(0,1) inputs, 4096^3.

    Tolerance: 1e-5 relative.  The matrix-core kernel (the default) sums k in the instruction's
    order, so it is held to the two forms of "relative" that are meaningful for a dot product
    whose terms cancel: |d - r| <= 1e-5 * sum_k |a||b| for every element, and
    ||d - r||_F <= 1e-5 * ||r||_F for the matrix.  (An element-wise bound against |r| itself is
    not attainable for any change of summation order where the terms cancel to |r| ~ 1.)
    The vector-ALU tile sums in the host reference's order and is bit-exact."""
    from cuasr_amd import inputs
    n = 4096
    A, B = inputs.normal(601, n, n), inputs.normal(602, n, n)
    C = np.zeros((n, n), dtype=np.float32, order="F")
    want = oracle.srgemm("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0)
    assert_same_bits(_run("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0, 1.0, "f32", "direct"), want, "vector-ALU plus-times")
    got = _run("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0, 1.0, "f32")
    diff = got.astype(np.float64) - want.astype(np.float64)
    import torch
    # sum_k |a||b| for every element (a bound, so torch's own fp32 product is accurate enough)
    mag = (torch.from_numpy(np.abs(A)).cuda() @ torch.from_numpy(np.abs(B)).cuda()).cpu().numpy().astype(np.float64)
    assert np.all(np.abs(diff) <= 1e-5 * mag)
    assert np.linalg.norm(diff) <= 1e-5 * np.linalg.norm(want.astype(np.float64))
    big = np.abs(want) >= 1.0
    print("fp32 plus-times 4096^3: max relative error over |r| >= 1:", float((np.abs(diff[big]) / np.abs(want[big])).max()))


def test_config5b_plus_times_f64_4096(oracle, lib):
    """The fp64 analogue of the plus-times control: N(0,1) inputs, 4096^3, tolerance 1e-12 relative
    (per element against sum_k |a||b|, and in the Frobenius norm); the vector-ALU tile bit-exact."""
    import torch
    from cuasr_amd import inputs
    n = 4096
    A = inputs.normal(611, n, n).astype(np.float64, order="F") + 2.0 ** -30 * inputs.normal(613, n, n).astype(np.float64, order="F")
    B = inputs.normal(612, n, n).astype(np.float64, order="F") + 2.0 ** -30 * inputs.normal(614, n, n).astype(np.float64, order="F")
    C = np.zeros((n, n), dtype=np.float64, order="F")
    want = oracle.srgemm("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0)
    assert_same_bits(_run("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0, 1.0, "f64", "valu"), want, "vector-ALU fp64 plus-times")
    got = _run("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0, 1.0, "f64")
    diff = np.abs(got - want)
    mag = (torch.from_numpy(np.abs(A)).cuda() @ torch.from_numpy(np.abs(B)).cuda()).cpu().numpy()
    assert np.all(diff <= 1e-12 * mag)
    assert np.linalg.norm(diff) <= 1e-12 * np.linalg.norm(want)
    big = np.abs(want) >= 1.0
    print("fp64 plus-times 4096^3: max relative error over |r| >= 1:", float((diff[big] / np.abs(want[big])).max()))
