"""Contract details of the operator boundary, on the GPU and through the C ABI: device-resident
alpha / beta, D aliasing C, launches on a caller's stream, and the shapes the reference's
cross-implementation tests use (test/regress/Srgemm_test.cu:118-605: tall-skinny, short-wide,
sub-matrices of larger buffers)."""
import numpy as np
import pytest

from helpers import assert_same_bits, to_device, to_host

pytestmark = pytest.mark.gpu

FAMILIES = ["naive", "valu", "direct", "mfma"]


def _inputs(m, n, k, seed=5):
    from cuasr_amd import inputs
    A = inputs.integers(seed, m, k, -8, 8, np.float32, "F")
    B = inputs.integers(seed + 1, k, n, -8, 8, np.float32, "F")
    C = inputs.integers(seed + 2, m, n, -8, 8, np.float32, "F")
    return A, B, C


@pytest.mark.parametrize("kernel", FAMILIES)
def test_alpha_beta_from_device_memory(oracle, lib, kernel):
    """alpha_ptr / beta_ptr override the immediate scalars (semiring_linear_combination.h:88-99, :112-115),
    and whether C is read is decided on the device from the pointed-to beta (:118-125)."""
    import torch
    import cuasr_amd
    m, n, k = 256, 128, 96
    A, B, C = _inputs(m, n, k)
    inf = np.float32(np.inf)
    for beta in (np.float32(0.0), inf):          # min-plus one (C is read) and zero (C is not read)
        want = oracle.srgemm("minimum", "plus", A, B, C, 2.0, beta, inf)
        d_alpha = torch.tensor([2.0], dtype=torch.float32, device="cuda")
        d_beta = torch.tensor([float(beta)], dtype=torch.float32, device="cuda")
        dD = to_device(np.zeros_like(C))
        # the immediate scalars are deliberately wrong: the pointers must win
        cuasr_amd.srgemm("minimum", "plus", to_device(A), to_device(B), to_device(C), dD, 7.0, 3.0, float("inf"), 0.0,
                         kernel=kernel, alpha_ptr=d_alpha.data_ptr(), beta_ptr=d_beta.data_ptr())
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, "f32"), want, f"{kernel} beta={beta}")
        if beta == inf:
            # C is not needed: a null C must be accepted and never dereferenced
            dD2 = to_device(np.zeros_like(C))
            cuasr_amd.srgemm("minimum", "plus", to_device(A), to_device(B), None, dD2, 2.0, float("inf"), float("inf"), 0.0,
                             kernel=kernel)
            torch.cuda.synchronize()
            assert_same_bits(to_host(dD2, "f32"), want, f"{kernel} null C")


@pytest.mark.parametrize("kernel", FAMILIES)
@pytest.mark.parametrize("layout", ["F", "C"])
def test_d_may_alias_c(oracle, lib, kernel, layout):
    """D = C in place (examples/00_minplus_srgemm/minplus_srgemm.cu:79-80)."""
    import torch
    import cuasr_amd
    m, n, k = 384, 256, 64
    A, B, C = _inputs(m, n, k, seed=11)
    A, B, C = (np.asarray(x, order=layout) for x in (A, B, C))
    want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf)
    dC = to_device(C)
    cuasr_amd.srgemm("minimum", "plus", to_device(A), to_device(B), dC, dC, 0.0, 0.0, float("inf"), 0.0, kernel=kernel)
    torch.cuda.synchronize()
    assert_same_bits(np.asarray(to_host(dC, "f32"), order=layout), want, kernel)


def test_launch_on_callers_stream(oracle, lib):
    """Calls are asynchronous on the stream they are given and ordered by it: a chain of dependent
    squarings on a side stream, with unrelated work on the default stream in between."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    n = 512
    D0 = inputs.graph_distances(77, n, density=0.05)
    host = D0
    for _ in range(4):
        host = oracle.srgemm("minimum", "plus", host, host, host, 0.0, 0.0, np.inf)
    side = torch.cuda.Stream()
    bufs = [to_device(D0), to_device(np.zeros_like(D0)), to_device(np.zeros_like(D0))]
    torch.cuda.synchronize()
    cur = bufs[0]
    noise = torch.zeros(1 << 20, device="cuda")
    for i in range(4):
        dst = bufs[1 + (i & 1)]
        cuasr_amd.srgemm("minimum", "plus", cur, cur, cur, dst, 0.0, 0.0, float("inf"), 0.0, stream=side)
        noise += 1.0  # default stream, independent
        cur = dst
    side.synchronize()
    assert_same_bits(to_host(cur, "f32"), host, "4 squarings on a side stream")
    torch.cuda.synchronize()
    assert float(noise[0]) == 4.0


@pytest.mark.parametrize("shape", [(125, 125, 1000), (1000, 1000, 125), (1, 1000, 1000), (1000, 1, 1000), (1000, 1000, 1),
                                   (3, 5, 7)])
@pytest.mark.parametrize("kernel", ["auto", "valu", "naive"])
def test_reference_cross_implementation_shapes(oracle, lib, shape, kernel):
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m, n, k = shape
    A = inputs.uniform(21, m, k, 1.5, 100.0)
    B = inputs.uniform(22, k, n, 1.5, 100.0)
    C = inputs.uniform(23, m, n, 1.5, 100.0)
    want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf)
    dD = to_device(np.zeros_like(C))
    cuasr_amd.srgemm("minimum", "plus", to_device(A), to_device(B), to_device(C), dD, 0.0, 0.0, float("inf"), 0.0, kernel=kernel)
    torch.cuda.synchronize()
    assert_same_bits(to_host(dD, "f32"), want, f"{shape} {kernel}")


def test_calls_can_be_captured_in_a_graph(oracle, lib):
    """Nothing in a call allocates, frees or synchronises, so a stream capture may contain it: two squarings, a
    parallel and a serial split-K are captured once and replayed on new inputs, with eager work and
    synchronisations between the replays; every replay must equal the eager result."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    n, k = 192, 640
    inf = float("inf")
    d_in = torch.empty(n, n, device="cuda").t()            # column-major, as the repeated-squaring step uses it
    d_mid, d_out = torch.empty(n, n, device="cuda").t(), torch.empty(n, n, device="cuda").t()
    a = torch.empty(n, k, device="cuda")                    # k contiguous in both operands: the split-K example's layout
    b = torch.empty(n, k, device="cuda").t()
    s_par, s_ser = torch.empty(n, n, device="cuda"), torch.empty(n, n, device="cuda")
    ws = torch.empty(n * n * 4, dtype=torch.float32, device="cuda")

    def work():
        cuasr_amd.srgemm("minimum", "plus", d_in, d_in, d_in, d_mid, 0.0, 0.0, inf, 0.0)
        cuasr_amd.srgemm("minimum", "plus", d_mid, d_mid, d_mid, d_out, 0.0, 0.0, inf, 0.0)
        cuasr_amd.srgemm_splitk("minimum", "plus", a, b, d_out.t(), s_par, 4, ws, 0.0, 0.0, inf, 0.0)
        cuasr_amd.srgemm_splitk_serial("minimum", "plus", a, b, d_out.t(), s_ser, 3, ws, 0.0, 0.0, inf, 0.0)

    def load(seed):
        D = inputs.graph_distances(seed, n, density=0.2, lo=1.0, hi=9.0)
        A, B = inputs.uniform(seed + 1, n, k, 0.0, 10.0, order="C"), inputs.uniform(seed + 2, k, n, 0.0, 10.0, order="F")
        d_in.copy_(torch.from_numpy(np.ascontiguousarray(D.T)).cuda().t())
        a.copy_(torch.from_numpy(A).cuda())
        b.copy_(torch.from_numpy(np.ascontiguousarray(B.T)).cuda().t())
        return D, A, B

    load(100)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        work()
    for seed in (200, 300, 400):
        D, A, B = load(seed)
        # eager work of the program's own between the replays
        scratch = torch.rand(256, 256, device="cuda") @ torch.rand(256, 256, device="cuda")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        del scratch
        D1 = oracle.srgemm("minimum", "plus", D, D, D, 0.0, 0.0, np.inf)
        D2 = oracle.srgemm("minimum", "plus", D1, D1, D1, 0.0, 0.0, np.inf)
        assert_same_bits(d_out.cpu().numpy(), D2, f"graph replay, seed {seed}: squarings")
        C = np.ascontiguousarray(D2.T)                      # d_out.t() is the transpose, row-major
        want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf)
        assert_same_bits(s_par.cpu().numpy(), want, f"graph replay, seed {seed}: split-K")
        assert_same_bits(s_ser.cpu().numpy(), want, f"graph replay, seed {seed}: serial split-K")


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("serial", [False, True])
def test_splitk_workspace_aligned_to_the_element_only(oracle, lib, dtype, serial):
    """A split-K workspace at an element boundary that is not a 16-byte boundary: the descriptor is one the
    direct-to-LDS tile is chosen for (1024 x 1024 x 4096 in 16 slices fills its rounds, operands aligned),
    so AUTO has to notice the workspace and fall back to a family that stores element-wise."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    npd = {"f32": np.float32, "f64": np.float64}[dtype]
    m, n, k, slices = 1024, 1024, 4096, 16
    A = inputs.uniform(61, m, k, 0.0, 10.0, npd, "F")
    B = inputs.uniform(62, k, n, 0.0, 10.0, npd, "F")
    C = inputs.uniform(63, m, n, 0.0, 10.0, npd, "F")
    want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf)   # min is order-free: both split-K forms equal the plain product
    es = np.dtype(npd).itemsize
    nbytes = cuasr_amd.splitk_workspace_bytes(m, n, slices, dtype)
    raw = torch.empty(nbytes + 16, dtype=torch.uint8, device="cuda")
    assert raw.data_ptr() % 16 == 0
    run = cuasr_amd.srgemm_splitk_serial if serial else cuasr_amd.srgemm_splitk
    import ctypes
    for offset in (0, es):
        dD = to_device(np.zeros_like(C))
        desc = cuasr_amd.make_desc("minimum", "plus", dtype, to_device(A), to_device(B), to_device(C), dD, 0.0, 0.0, float("inf"), 0.0, slices)
        assert lib.cuasr_amd_selected_kernel(ctypes.byref(desc)) == b"valu_direct"   # what the operands alone would get
        run("minimum", "plus", to_device(A), to_device(B), to_device(C), dD, slices, raw.data_ptr() + offset,
            0.0, 0.0, float("inf"), 0.0, dtype=dtype)
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, dtype), want, f"{dtype} workspace offset {offset}")


def test_reduction_kernel_on_its_own(oracle, lib):
    """cuasr_amd_reduce_splitk folds partial tiles that are already in the workspace: after a split-K call it
    reproduces that call's output into another D, and on hand-made partial tiles it gives their fold
    (reduction/kernel/reduce_split_k.h:162-227: slices in ascending order, then the epilogue with C)."""
    import ctypes
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m, n, k, slices = 200, 120, 1040, 5
    A = inputs.uniform(71, m, k, 0.0, 10.0, np.float32, "C")
    B = inputs.uniform(72, k, n, 0.0, 10.0, np.float32, "C")
    C = inputs.uniform(73, m, n, 0.0, 10.0, np.float32, "C")
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    ws = torch.empty(slices * m * n, dtype=torch.float32, device="cuda")
    d1, d2 = to_device(np.zeros_like(C)), to_device(np.zeros_like(C))
    cuasr_amd.srgemm_splitk("minimum", "plus", dA, dB, dC, d1, slices, ws, 0.0, 0.0, float("inf"), 0.0)
    desc = cuasr_amd.make_desc("minimum", "plus", "f32", dA, dB, dC, d2, 0.0, 0.0, float("inf"), 0.0, slices)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.cuasr_amd_reduce_splitk(ctypes.byref(desc), ctypes.c_void_p(ws.data_ptr()), stream) == 0
    torch.cuda.synchronize()
    want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf)
    assert_same_bits(to_host(d1, "f32"), want, "split-K")
    assert_same_bits(to_host(d2, "f32"), want, "reduction alone")
    # hand-made partial tiles (row-major output: slice z at ws + z * m * n): D = min(min_z partial_z, C)
    parts = np.stack([inputs.uniform(80 + z, m, n, 0.0, 10.0, np.float32, "C") for z in range(slices)])
    ws.copy_(torch.from_numpy(parts.reshape(-1)).cuda())
    assert lib.cuasr_amd_reduce_splitk(ctypes.byref(desc), ctypes.c_void_p(ws.data_ptr()), stream) == 0
    torch.cuda.synchronize()
    assert_same_bits(to_host(d2, "f32"), np.minimum(parts.min(axis=0), C), "hand-made partial tiles")


def test_a_callers_pending_error_does_not_fail_a_good_launch(oracle, lib):
    """A launch reports its own status: an error an earlier runtime call of the caller left on this thread
    (here hipErrorNotReady from querying a busy stream) must not make a good launch read as a failure."""
    import ctypes
    import torch
    import cuasr_amd
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipStreamQuery.argtypes = [ctypes.c_void_p]
    A, B, C = _inputs(256, 256, 512)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD = to_device(np.zeros_like(C))
    big = torch.rand(8192, 8192, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    hip.hipGetLastError()                      # start clean
    pending = 0
    for _ in range(20):                        # keep the stream busy, then ask whether it is done
        torch.mm(big, big)
        pending = hip.hipStreamQuery(ctypes.c_void_p(stream))
        if pending != 0:
            break
    if pending == 0:
        pytest.skip("the stream never reported hipErrorNotReady")
    for kernel in ("direct", "valu", "naive"):
        cuasr_amd.srgemm("minimum", "plus", dA, dB, dC, dD, 0.0, 0.0, float("inf"), 0.0, kernel=kernel)   # raises on any status but success
    torch.cuda.synchronize()
    assert_same_bits(to_host(dD, "f32"), oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf), "after a pending error")
