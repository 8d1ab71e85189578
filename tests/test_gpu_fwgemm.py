"""GPU parity of the min-plus product with predecessor tracking and of the
repeated-squaring driver, through the C ABI, against the CPU oracle
(test/regress/include/fwgpu/cpu_srgemm.hpp:20-48).  Distances are compared
bit for bit, parents exactly."""
import numpy as np
import pytest

import cuasr_amd
from cuasr_amd import inputs
from helpers import assert_same_bits, to_device

pytestmark = pytest.mark.gpu


def operands(seed, m, n, k, dtype, ties, pad=(0, 0, 0, 0), inf_share=0.2):
    """Column-major A, B, dist, parent as views with the given extra leading-dimension rows."""
    rng = np.random.default_rng(seed)
    def mat(r, c, lo, hi, extra):
        buf = np.full((r + extra, c), 1.0, dtype=dtype, order="F")
        v = rng.integers(lo, hi, (r, c)).astype(dtype) if ties else (rng.random((r, c)) * 10).astype(dtype)
        v[rng.random((r, c)) < inf_share] = np.inf
        buf[:r] = v
        return buf
    A, B = mat(m, k, 0, 6, pad[0]), mat(k, n, 0, 6, pad[1])
    dist = mat(m, n, 2, 9, pad[2])
    parent = np.full((m + pad[3], n), -7, dtype=np.int32, order="F")
    return A, B, dist, parent


def run_case(oracle, m, n, k, dtype, ties, kernel, pad=(0, 0, 0, 0), seed=0):
    A, B, dist, parent = operands(seed + m + 3 * n + 5 * k, m, n, k, dtype, ties, pad)
    dA, dB, dD, dP = (to_device(x) for x in (A, B, dist, parent))
    cuasr_amd.fwgemm(dA[:m], dB[:k], dD[:m], dP[:m], kernel=kernel)
    want_d, want_p = dist.copy(order="F"), parent.copy(order="F")
    oracle.fwgemm(A[:m], B[:k], want_d[:m], want_p[:m])
    got_d, got_p = dD.cpu().numpy(), dP.cpu().numpy()
    what = f"{np.dtype(dtype).name} {m}x{n}x{k} {kernel} ties={ties} pad={pad}"
    assert_same_bits(got_d, want_d, "dist " + what)          # rows beyond m (the padding) untouched as well
    bad = np.argwhere(got_p != want_p)
    assert len(bad) == 0, f"parent {what}: {len(bad)} differ, first {bad[0]}: {got_p[tuple(bad[0])]} != {want_p[tuple(bad[0])]}"
    return want_p[:m]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("kernel", ["naive", "valu"])
@pytest.mark.parametrize("ties", [True, False])
def test_whole_tiles(oracle, dtype, kernel, ties):
    for m, n, k in [(128, 128, 64), (256, 384, 160), (128, 256, 16)]:
        p = run_case(oracle, m, n, k, dtype, ties, kernel)
        assert (p == -7).any() and (p >= 0).any()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("kernel", ["naive", "valu", "auto"])
def test_ragged_extents_and_leading_dimensions(oracle, dtype, kernel):
    for m, n, k in [(1, 1, 1), (5, 7, 3), (129, 127, 17), (200, 130, 95), (63, 300, 33), (257, 65, 1)]:
        run_case(oracle, m, n, k, dtype, True, kernel)
        run_case(oracle, m, n, k, dtype, False, kernel, pad=(3, 1, 2, 5))
    # whole tiles, but leading dimensions that break the vector alignment
    run_case(oracle, 128, 128, 32, dtype, True, kernel, pad=(1, 2, 0, 0))
    run_case(oracle, 128, 128, 32, dtype, True, kernel, pad=(4, 4, 8, 12))


def test_first_of_many_equal_products(oracle):
    """Every product equal: the first k wins where it improves, nothing moves where it does not."""
    m = n = 128
    k = 96
    A = np.ones((m, k), np.float32, order="F")
    B = np.ones((k, n), np.float32, order="F")
    dist = np.asfortranarray(np.where(np.add.outer(np.arange(m), np.arange(n)) % 2 == 0, 5.0, 2.0).astype(np.float32))
    parent = np.full((m, n), -1, np.int32, order="F")
    dA, dB, dD, dP = (to_device(x) for x in (A, B, dist, parent))
    cuasr_amd.fwgemm(dA, dB, dD, dP, kernel="valu")
    got_d, got_p = dD.cpu().numpy(), dP.cpu().numpy()
    assert np.array_equal(got_d, np.full((m, n), 2.0, np.float32))
    assert np.array_equal(got_p, np.where(dist == 5.0, 0, -1))
    # the minimum sits in a later chunk for some elements and is met again afterwards
    A[:, :40] = 3.0
    A[::2, 70] = 0.5
    dA, dD, dP = to_device(A), to_device(dist), to_device(parent)
    cuasr_amd.fwgemm(dA, dB, dD, dP, kernel="valu")
    want_d, want_p = dist.copy(order="F"), parent.copy(order="F")
    oracle.fwgemm(A, B, want_d, want_p)
    assert_same_bits(dD.cpu().numpy(), want_d, "dist")
    assert np.array_equal(dP.cpu().numpy(), want_p)
    assert set(np.unique(want_p)) == {-1, 40, 70}


def test_signed_zero_products(oracle):
    """A product that is -0 does not beat a +0 found earlier (and the other way round); the stored
    distance is the first of them, as in the sequential scan."""
    m, n, k = 128, 128, 32
    rng = np.random.default_rng(5)
    A = np.asfortranarray(rng.choice(np.array([0.0, -0.0, 1.0], np.float32), (m, k)))
    B = np.asfortranarray(rng.choice(np.array([0.0, -0.0, 2.0], np.float32), (k, n)))
    dist = np.full((m, n), 1.0, np.float32, order="F")
    parent = np.full((m, n), -1, np.int32, order="F")
    for kernel in ("naive", "valu"):
        dA, dB, dD, dP = (to_device(x) for x in (A, B, dist, parent))
        cuasr_amd.fwgemm(dA, dB, dD, dP, kernel=kernel)
        want_d, want_p = dist.copy(order="F"), parent.copy(order="F")
        oracle.fwgemm(A, B, want_d, want_p)
        assert_same_bits(dD.cpu().numpy(), want_d, "dist " + kernel)
        assert np.array_equal(dP.cpu().numpy(), want_p)
    assert np.signbit(want_d).any() and (~np.signbit(want_d)).any()


def test_large_square_step_properties():
    """4096^3 (the size of the headline workload): too large for the CPU scan, so check what the
    definition fixes -- dist equals the min-plus SRGEMM bit for bit, improved elements carry a parent
    whose product is the new distance and no earlier k gives it, others keep distance and parent."""
    import torch
    n = 4096
    D = inputs.graph_distances(3, n)
    dA = to_device(D)
    dD, dP = dA.clone(), torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    cuasr_amd.fwgemm(dA, dA, dD, dP)
    ref = torch.empty_like(dA)
    cuasr_amd.srgemm("minimum", "plus", dA, dA, dA, ref, alpha=0.0, beta=0.0, add_identity=float("inf"))
    assert torch.equal(dD, ref)
    improved = dD < dA
    assert torch.equal(dP >= 0, improved)
    rows, cols = torch.nonzero(improved, as_tuple=True)
    pick = torch.randperm(rows.numel(), device="cuda")[:20000]
    r, c = rows[pick], cols[pick]
    p = dP[r, c].long()
    assert torch.equal(dA[r, p] + dA[p, c], dD[r, c])
    # no smaller k reaches the same value: compare with the first-occurrence argmin over all k
    first = torch.stack([(dA[ri, :] + dA[:, ci]).eq(dD[ri, ci]).nonzero()[0, 0] for ri, ci in zip(r[:200], c[:200])])
    assert torch.equal(first, p[:200])


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [300, 256])   # ragged tiles; whole, aligned tiles (the vector lookup in the transposed snapshot)
def test_apsp_squaring_rebuilds_shortest_paths(oracle, n, dtype):
    import torch
    from scipy.sparse.csgraph import floyd_warshall as scipy_fw
    rng = np.random.default_rng(21 + n)
    W = np.where(rng.random((n, n)) < 0.03, rng.integers(1, 50, (n, n)), np.inf).astype(dtype)
    np.fill_diagonal(W, 0)
    dD = to_device(np.asfortranarray(W))
    dP = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    ws = torch.empty(cuasr_amd.apsp_workspace_bytes(n, "f32" if dtype == np.float32 else "f64"), dtype=torch.uint8, device="cuda")
    cuasr_amd.apsp_squaring(dD, dP, ws)
    dist, parent = dD.cpu().numpy(), dP.cpu().numpy()
    assert np.array_equal(dist.astype(np.float64), scipy_fw(W.astype(np.float64)))
    # the same iterations on the CPU give the same parents
    want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    for _ in range(int(np.ceil(np.log2(n - 1)))):
        snap = want_d.copy(order="F")
        oracle.fwgemm(snap, snap, want_d, want_p)
    assert_same_bits(dist, want_d, "dist")
    assert np.array_equal(parent, want_p)

    def expand(i, j):
        k = parent[i, j]
        return [] if k < 0 else expand(i, k) + [int(k)] + expand(k, j)
    rng2 = np.random.default_rng(1)
    for i, j in rng2.integers(0, n, (300, 2)):
        if i == j or np.isinf(dist[i, j]):
            assert parent[i, j] == -1
            continue
        hops = [i] + expand(i, j) + [j]
        assert sum(W[a, b] for a, b in zip(hops, hops[1:])) == dist[i, j]


def _check_paths(W, dist, parent, seed, count=300):
    n = W.shape[0]

    def expand(i, j):
        k = parent[i, j]
        return [] if k < 0 else expand(i, k) + [int(k)] + expand(k, j)
    rng = np.random.default_rng(seed)
    for i, j in rng.integers(0, n, (count, 2)):
        if i == j or np.isinf(dist[i, j]):
            assert parent[i, j] == -1
            continue
        hops = [i] + expand(i, j) + [j]
        assert sum(W[a, b] for a, b in zip(hops, hops[1:])) == dist[i, j]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,pad", [(1, 0), (100, 0), (128, 0), (300, 3), (384, 0), (513, 1),
                                   # 128 tiles and more: the tiled product with the block row / column tiles skipped
                                   (1536, 0), (1500, 4), (1475, 1)])
def test_apsp_blocked_floyd_warshall(oracle, n, pad, dtype):
    """Blocked Floyd-Warshall: distances equal to scipy's on integer weights (every order of
    additions is exact), dist and parent bit-identical to the oracle's blocked iteration, and the
    paths rebuilt from parent sum to the distances."""
    import torch
    from scipy.sparse.csgraph import floyd_warshall as scipy_fw
    rng = np.random.default_rng(77 + n)
    W = np.where(rng.random((n, n)) < max(0.02, 3.0 / n), rng.integers(1, 60, (n, n)), np.inf).astype(dtype)
    np.fill_diagonal(W, 0)
    host = np.full((n + pad, n), 7.0, dtype=dtype, order="F")     # leading dimension n + pad
    host[:n] = W
    dD = to_device(host)
    dP = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    name = "f32" if dtype == np.float32 else "f64"
    ws = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(n, name), dtype=torch.uint8, device="cuda")
    cuasr_amd.apsp_blocked(dD[:n], dP, ws)
    got, parent = dD.cpu().numpy(), dP.cpu().numpy()
    assert (got[n:] == 7.0).all()                                # the padding rows are untouched
    dist = got[:n]
    assert np.array_equal(dist.astype(np.float64), scipy_fw(W.astype(np.float64)))
    want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    oracle.apsp_blocked(want_d, want_p, 128)
    assert_same_bits(np.ascontiguousarray(dist), np.ascontiguousarray(want_d), "dist")
    assert np.array_equal(parent, want_p)
    _check_paths(W, dist, parent, n)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_apsp_blocked_keeps_the_sign_of_a_zero(oracle, dtype):
    """Edges of weight +0 and -0: a sum of two -0 is -0, and the strict comparison keeps whichever zero was
    there first, where a hardware minimum would prefer -0.  The diagonal blocks that hold a -0 are closed by
    comparison and select; dist (bit for bit, so with its signs) and parent equal the oracle's."""
    import torch
    n = 1475
    rng = np.random.default_rng(4242)
    W = np.where(rng.random((n, n)) < 0.004, rng.integers(1, 9, (n, n)), np.inf).astype(dtype)
    zeros = rng.random((n, n)) < 0.004
    W[zeros] = rng.choice(np.array([0.0, -0.0], dtype), int(zeros.sum()))
    # every diagonal block but the fourth has a -0 of its own
    W[128 * 3:128 * 4, 128 * 3:128 * 4][W[128 * 3:128 * 4, 128 * 3:128 * 4] == 0] = 0.0
    np.fill_diagonal(W, 0)
    assert np.signbit(W[W == 0]).any()
    dD = to_device(np.asfortranarray(W))
    dP = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    name = "f32" if dtype == np.float32 else "f64"
    ws = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(n, name), dtype=torch.uint8, device="cuda")
    cuasr_amd.apsp_blocked(dD, dP, ws)
    want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    oracle.apsp_blocked(want_d, want_p, 128)
    dist = dD.cpu().numpy()
    assert np.signbit(want_d[want_d == 0]).any() and not np.signbit(want_d[want_d == 0]).all()
    assert_same_bits(np.ascontiguousarray(dist), np.ascontiguousarray(want_d), "dist")
    assert np.array_equal(dP.cpu().numpy(), want_p)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,pad", [(100, 0), (384, 0), (513, 1), (700, 4), (1475, 1)])
def test_apsp_blocked_with_tiled_panels(oracle, n, pad, dtype):
    """The way a block step updates its block row and column from n = 16257 on (two launches of the tiled
    kernel with the diagonal block skipped, then a transposing copy of the column), forced at sizes the
    oracle can run: dist and parent bit-identical to the oracle and to the paired form."""
    import torch
    rng = np.random.default_rng(177 + n)
    W = np.where(rng.random((n, n)) < max(0.02, 3.0 / n), rng.random((n, n)) * 9 + 0.5, np.inf).astype(dtype)   # sums round
    np.fill_diagonal(W, 0)
    host = np.full((n + pad, n), 7.0, dtype=dtype, order="F")
    host[:n] = W
    name = "f32" if dtype == np.float32 else "f64"
    results = {}
    for panels in ("tiled", "paired"):
        dD = to_device(host)
        dP = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
        ws = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(n, name), dtype=torch.uint8, device="cuda")
        cuasr_amd.apsp_blocked(dD[:n], dP, ws, panels=panels)
        got = dD.cpu().numpy()
        assert (got[n:] == 7.0).all()
        results[panels] = (np.ascontiguousarray(got[:n]), dP.cpu().numpy())
    want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    oracle.apsp_blocked(want_d, want_p, 128)
    for panels, (dist, parent) in results.items():
        assert_same_bits(dist, np.ascontiguousarray(want_d), f"dist, {panels} panels")
        assert np.array_equal(parent, want_p), panels


def test_apsp_blocked_on_rounding_weights_matches_the_oracle_bit_for_bit(oracle):
    """Real-valued weights: sums round, so the result depends on the order of additions; the
    device and the oracle use the same order.  Against repeated squaring only closeness holds."""
    import torch
    n = 640
    rng = np.random.default_rng(5)
    W = np.where(rng.random((n, n)) < 0.02, rng.random((n, n)) * 10 + 0.1, np.inf).astype(np.float32)
    np.fill_diagonal(W, 0)
    dD = to_device(np.asfortranarray(W))
    dP = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    ws = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(n, "f32"), dtype=torch.uint8, device="cuda")
    cuasr_amd.apsp_blocked(dD, dP, ws)
    want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    oracle.apsp_blocked(want_d, want_p, 128)
    dist, parent = dD.cpu().numpy(), dP.cpu().numpy()
    assert_same_bits(np.ascontiguousarray(dist), np.ascontiguousarray(want_d), "dist")
    assert np.array_equal(parent, want_p)
    sq = to_device(np.asfortranarray(W))
    sqp = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    ws2 = torch.empty(cuasr_amd.apsp_workspace_bytes(n, "f32"), dtype=torch.uint8, device="cuda")
    cuasr_amd.apsp_squaring(sq, sqp, ws2)
    ref = sq.cpu().numpy()
    finite = np.isfinite(ref)
    assert np.array_equal(finite, np.isfinite(dist))
    assert np.allclose(dist[finite], ref[finite], rtol=1e-5, atol=0)
    # paths rebuilt from parent are real paths of (almost) the recorded length
    def expand(i, j):
        k = parent[i, j]
        return [] if k < 0 else expand(i, k) + [int(k)] + expand(k, j)
    for i, j in rng.integers(0, n, (200, 2)):
        if i == j or not finite[i, j]:
            continue
        hops = [i] + expand(i, j) + [j]
        assert abs(sum(float(W[a, b]) for a, b in zip(hops, hops[1:])) - dist[i, j]) <= 1e-4 * dist[i, j]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n", [1536, 1501])
def test_apsp_squaring_two_steps_on_the_tiled_kernel(oracle, n, dtype):
    """Outputs of 128 tiles and more run on the tiled kernel, whose search for the first
    minimising k reads the transposed snapshot: two squarings, dist and parent bit for bit."""
    import torch
    rng = np.random.default_rng(n)
    W = np.where(rng.random((n, n)) < 0.01, rng.integers(1, 9, (n, n)), np.inf).astype(dtype)   # many ties
    np.fill_diagonal(W, 0)
    dD = to_device(np.asfortranarray(W))
    dP = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    ws = torch.empty(cuasr_amd.apsp_workspace_bytes(n, "f32" if dtype == np.float32 else "f64"), dtype=torch.uint8, device="cuda")
    cuasr_amd.apsp_squaring(dD, dP, ws, iterations=2)
    want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    for _ in range(2):
        snap = want_d.copy(order="F")
        oracle.fwgemm(snap, snap, want_d, want_p)
    assert_same_bits(np.ascontiguousarray(dD.cpu().numpy()), np.ascontiguousarray(want_d), "dist")
    assert np.array_equal(dP.cpu().numpy(), want_p)


@pytest.mark.parametrize("n,squarings", [(1280, 3), (2048, 1)])
def test_apsp_squaring_on_the_direct_tile(oracle, n, squarings):
    """Whole tiles of 128 x 256 with k in whole chunks of 32 (fp32) take the predecessor-tracking product on the
    hand-scheduled direct-to-LDS tile: real-valued weights (sums round, ties are rare) and a share of exact zeros
    (ties with the diagonal), dist and parent bit for bit after every squaring."""
    import torch
    rng = np.random.default_rng(900 + n)
    W = np.where(rng.random((n, n)) < 0.02, rng.random((n, n)) * 7 + 0.25, np.inf).astype(np.float32)
    W[rng.random((n, n)) < 0.002] = 0.0
    np.fill_diagonal(W, 0)
    dD = to_device(np.asfortranarray(W))
    dP = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
    ws = torch.empty(cuasr_amd.apsp_workspace_bytes(n, "f32"), dtype=torch.uint8, device="cuda")
    want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    for s in range(squarings):
        cuasr_amd.apsp_squaring(dD, dP, ws, iterations=1)
        snap = want_d.copy(order="F")
        oracle.fwgemm(snap, snap, want_d, want_p)
        assert_same_bits(np.ascontiguousarray(dD.cpu().numpy()), np.ascontiguousarray(want_d), f"dist after squaring {s + 1}")
        assert np.array_equal(dP.cpu().numpy(), want_p), f"parent after squaring {s + 1}"


def test_apsp_4096_blocked_and_squaring_agree():
    """Full size, integer weights (every order of additions exact): blocked Floyd-Warshall and
    repeated squaring are different algorithms and must find the same distances; both parent
    matrices must describe paths of exactly those lengths; squaring once more changes nothing."""
    import torch
    n = 4096
    rng = np.random.default_rng(4096)
    W = np.where(rng.random((n, n)) < 0.002, rng.integers(1, 100, (n, n)), np.inf).astype(np.float32)
    np.fill_diagonal(W, 0)
    dW = to_device(np.asfortranarray(W))
    results = []
    for solver, size in ((cuasr_amd.apsp_blocked, cuasr_amd.apsp_blocked_workspace_bytes),
                         (cuasr_amd.apsp_squaring, cuasr_amd.apsp_workspace_bytes)):
        d = dW.clone()                       # (clone keeps the column-major strides)
        p = torch.full((n, n), -1, dtype=torch.int32, device="cuda").t()
        ws = torch.empty(size(n, "f32"), dtype=torch.uint8, device="cuda")
        solver(d, p, ws)
        results.append((d, p, ws))
    (db, pb, _), (ds, ps, ws) = results
    assert torch.equal(db, ds)
    assert bool(torch.isfinite(db).float().mean() > 0.5)          # the graph is mostly connected
    # a fixed point: one more squaring step improves nothing
    before, pbefore = ds.clone(), ps.clone()
    cuasr_amd.apsp_squaring(ds, ps, ws, iterations=1)
    assert torch.equal(ds, before) and torch.equal(ps, pbefore)
    dist = db.cpu().numpy()
    for parent in (pb.cpu().numpy(), pbefore.cpu().numpy()):
        _check_paths(W, dist, parent, seed=9, count=400)


def test_apsp_drivers_can_be_captured_in_a_graph(oracle):
    """Neither driver allocates, frees, copies through the runtime or synchronises: a stream capture
    may contain them.  Both are captured once and replayed on new graphs, with eager work and
    synchronisations between the replays; every replay must equal the oracle bit for bit."""
    import torch
    n = 300
    src = torch.empty(n, n, device="cuda").t()
    d_blk, d_sq = torch.empty(n, n, device="cuda").t(), torch.empty(n, n, device="cuda").t()
    p_blk = torch.empty(n, n, dtype=torch.int32, device="cuda").t()
    p_sq = torch.empty(n, n, dtype=torch.int32, device="cuda").t()
    w_blk = torch.empty(cuasr_amd.apsp_blocked_workspace_bytes(n, "f32"), dtype=torch.uint8, device="cuda")
    w_sq = torch.empty(cuasr_amd.apsp_workspace_bytes(n, "f32"), dtype=torch.uint8, device="cuda")

    def work():
        d_blk.copy_(src); d_sq.copy_(src)
        p_blk.fill_(-1); p_sq.fill_(-1)
        cuasr_amd.apsp_blocked(d_blk, p_blk, w_blk)
        cuasr_amd.apsp_squaring(d_sq, p_sq, w_sq, iterations=3)

    def load(seed):
        rng = np.random.default_rng(seed)
        W = np.where(rng.random((n, n)) < 0.03, rng.random((n, n)) * 9 + 0.5, np.inf).astype(np.float32)
        np.fill_diagonal(W, 0)
        src.copy_(torch.from_numpy(np.ascontiguousarray(W.T)).cuda().t())
        return W

    load(1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        work()
    for seed in (2, 3, 4):
        W = load(seed)
        scratch = torch.rand(256, 256, device="cuda") @ torch.rand(256, 256, device="cuda")   # eager work in between
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        del scratch
        want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
        oracle.apsp_blocked(want_d, want_p, 128)
        assert_same_bits(np.ascontiguousarray(d_blk.cpu().numpy()), np.ascontiguousarray(want_d), f"blocked, seed {seed}")
        assert np.array_equal(p_blk.cpu().numpy(), want_p)
        want_d, want_p = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
        for _ in range(3):
            snap = want_d.copy(order="F")
            oracle.fwgemm(snap, snap, want_d, want_p)
        assert_same_bits(np.ascontiguousarray(d_sq.cpu().numpy()), np.ascontiguousarray(want_d), f"squaring, seed {seed}")
        assert np.array_equal(p_sq.cpu().numpy(), want_p)
