"""Edge cases through the C ABI: empty extents, extreme aspect ratios, and leading dimensions so large
that element offsets do not fit 32 bits."""
import numpy as np
import pytest

from helpers import assert_same_bits, to_device, to_host

pytestmark = pytest.mark.gpu

INF = float("inf")
NPD = {"f32": np.float32, "f64": np.float64, "u32": np.uint32}
# (add, mult, dtype, alpha, beta = one, beta = zero, add identity, mult identity)
SEMIRINGS = {
    "minplus_f32": ("minimum", "plus", "f32", 0.0, 0.0, INF, INF, 0.0),
    "maxplus_f64": ("maximum", "plus", "f64", 0.0, 0.0, -INF, -INF, 0.0),
    "plustimes_f64": ("plus", "multiplies", "f64", 1.0, 1.0, 0.0, 0.0, 1.0),
    "xorand_u32": ("bit_xor", "bit_and", "u32", 0xFFFFFFFF, 0xFFFFFFFF, 0, 0, 0xFFFFFFFF),
}


def operands(dtype, m, n, k, seed=5):
    from cuasr_amd import inputs
    if dtype == "u32":
        return inputs.words32(seed, m, k, "C"), inputs.words32(seed + 1, k, n, "F"), inputs.words32(seed + 2, m, n, "C")
    npd = NPD[dtype]
    return (inputs.integers(seed, m, k, -8, 8, npd, "C"), inputs.integers(seed + 1, k, n, -8, 8, npd, "F"),
            inputs.integers(seed + 2, m, n, -8, 8, npd, "C"))


@pytest.mark.parametrize("kernel", ["auto", "valu", "naive"])
@pytest.mark.parametrize("name", sorted(SEMIRINGS))
def test_no_terms_at_all(oracle, lib, name, kernel):
    """K = 0: the accumulator is the additive identity and the epilogue still runs (kernel/srgemm.h:220-225);
    M = 0 or N = 0: nothing to do, and nothing is touched."""
    import torch
    import cuasr_amd
    add, mult, dtype, alpha, one, zero, ident, mone = SEMIRINGS[name]
    m, n = 37, 29
    _, _, C = operands(dtype, m, n, 1)
    A = np.zeros((m, 0), dtype=NPD[dtype])
    B = np.zeros((0, n), dtype=NPD[dtype])
    tdt = {"f32": torch.float32, "f64": torch.float64, "u32": torch.int32}[dtype]
    dA = torch.empty(m, 1, dtype=tdt, device="cuda")[:, :0]   # m x 0, a valid pointer and leading dimension
    dB = torch.empty(n, 1, dtype=tdt, device="cuda")[:, :0].t()
    for beta in (one, zero):
        want = oracle.srgemm(add, mult, np.zeros((m, 1), NPD[dtype])[:, :0], np.zeros((1, n), NPD[dtype])[:0], C, alpha, beta, ident)
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm(add, mult, dA, dB, to_device(C), dD, alpha, beta, ident, mone, dtype=dtype, kernel=kernel)
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, dtype), want, f"K = 0 {name} {kernel} beta={beta}")
    # split-K over an empty k range: every slice holds the identity
    ws = torch.empty(4 * m * n * 2 + 4, dtype=torch.int32, device="cuda")
    want = oracle.srgemm(add, mult, np.zeros((m, 1), NPD[dtype])[:, :0], np.zeros((1, n), NPD[dtype])[:0], C, alpha, one, ident)
    for fn in (cuasr_amd.srgemm_splitk, cuasr_amd.srgemm_splitk_serial):
        dD = to_device(np.zeros_like(C))
        fn(add, mult, dA, dB, to_device(C), dD, 3, ws, alpha, one, ident, mone, dtype=dtype, kernel=kernel)
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, dtype), want, f"K = 0 split-K {name} {kernel} {fn.__name__}")
    # M = 0 / N = 0
    k = 16
    guard = torch.full((8, 8), 7, dtype=tdt, device="cuda")
    for mm, nn in ((0, 8), (8, 0), (0, 0)):
        a = torch.zeros(max(mm, 1), k, dtype=tdt, device="cuda")[:mm]
        b = torch.zeros(max(nn, 1), k, dtype=tdt, device="cuda")[:nn].t()
        d = guard[:mm, :nn]
        cuasr_amd.srgemm(add, mult, a, b, d, d, alpha, one, ident, mone, dtype=dtype, kernel=kernel)
        torch.cuda.synchronize()
    assert bool((guard == 7).all())


@pytest.mark.parametrize("kernel", ["auto", "valu", "naive"])
@pytest.mark.parametrize("shape", [(1, 1, 1 << 20), (70000, 3, 5), (3, 70000, 5), (2, 2, 65537), (1, 4096, 4096),
                                   (4096, 1, 4096), (5, 100000, 1), (100000, 4, 64)])
def test_extreme_aspect_ratios(oracle, lib, shape, kernel):
    import torch
    import cuasr_amd
    m, n, k = shape
    for name in ("minplus_f32", "maxplus_f64"):
        add, mult, dtype, alpha, one, zero, ident, mone = SEMIRINGS[name]
        A, B, C = operands(dtype, m, n, k)
        want = oracle.srgemm(add, mult, A, B, C, alpha, one, ident)
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm(add, mult, to_device(A), to_device(B), to_device(C), dD, alpha, one, ident, mone, dtype=dtype, kernel=kernel)
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, dtype), want, f"{name} {m}x{n}x{k} {kernel}")


@pytest.mark.parametrize("kernel", ["auto", "valu", "naive", "mfma"])
def test_leading_dimensions_beyond_32_bit_offsets(oracle, lib, kernel):
    """Rows 2^27 + 8 elements apart: the last row of each operand starts more than 2^32 bytes (and, for A, B and
    D in turn, more than 2^31 elements) past the first.  Addresses must be formed in 64 bits everywhere."""
    import torch
    import cuasr_amd
    ld = (1 << 27) + 8
    add, mult, dtype = ("plus", "multiplies", "f32") if kernel == "mfma" else ("minimum", "plus", "f32")
    ident, one = (0.0, 1.0) if kernel == "mfma" else (INF, 0.0)
    from cuasr_amd import inputs
    for m, n, k in ((20, 20, 36), (20, 16, 300)):
        A = inputs.integers(1, m, k, -8, 8, np.float32, "C")
        B = inputs.integers(2, k, n, -8, 8, np.float32, "F")
        C = inputs.integers(3, m, n, -8, 8, np.float32, "C")
        want = oracle.srgemm(add, mult, A, B, C, one, one, ident)

        def strided(host, rows, cols):  # rows `ld` elements apart in a buffer that is never initialised elsewhere
            buf = torch.empty((rows - 1) * ld + cols, dtype=torch.float32, device="cuda")
            view = buf.as_strided((rows, cols), (ld, 1))
            view.copy_(torch.from_numpy(np.ascontiguousarray(host)).cuda())
            return view

        dA = strided(A, m, k)               # row-major, lda = ld
        dB = strided(B.T, n, k).t()         # column-major, ldb = ld
        dC = strided(C, m, n)
        dD = strided(np.zeros_like(C), m, n)
        cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, one, one, ident, one, kernel=kernel)
        torch.cuda.synchronize()
        assert_same_bits(dD.cpu().numpy(), want, f"ld = 2^27 + 8, {m}x{n}x{k} {kernel}")
        del dA, dB, dC, dD
        torch.cuda.empty_cache()
