"""GPU parity of the batched call (a sequence of products sharing one descriptor) through the C ABI:
every product bit-identical to the oracle's SRGEMM on the same operands."""
import numpy as np
import pytest

import cuasr_amd
from helpers import assert_same_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", [
    ("minimum", "plus", np.float32, 0.0, 0.0, np.inf, 0.0),
    ("maximum", "minimum", np.float64, np.inf, np.inf, -np.inf, np.inf),
    ("plus", "multiplies", np.float64, 1.0, 1.0, 0.0, 1.0),
])
def test_batched_products_match_the_oracle(oracle, case):
    import torch
    add, mult, dtype, alpha, beta, ident, one = case
    batch, m, n, k = 5, 96, 80, 70
    rng = np.random.default_rng(17)
    # small integers: the plus-times sums are exact whatever their order
    A = rng.integers(0, 7, (batch, m, k)).astype(dtype)
    B = rng.integers(0, 7, (k, n)).astype(dtype)                      # one B for the whole batch (stride 0)
    C = rng.integers(0, 9, (batch, m, n + 3)).astype(dtype)           # padded rows: leading dimension n + 3
    dA = torch.from_numpy(A).cuda()
    dB = torch.from_numpy(B).cuda().unsqueeze(0).expand(batch, k, n)
    dC = torch.from_numpy(C).cuda()
    dD = torch.full((batch, m, n + 3), -5, dtype=dA.dtype, device="cuda")
    cuasr_amd.srgemm_batched(add, mult, dA, dB, dC[:, :, :n], dD[:, :, :n], alpha, beta, ident, one, kernel="valu")
    got = dD.cpu().numpy()
    assert (got[:, :, n:] == -5).all()                                 # the padding is untouched
    for i in range(batch):
        want = oracle.srgemm(add, mult, A[i], B, np.ascontiguousarray(C[i][:, :n]), alpha, beta, ident)
        assert_same_bits(np.ascontiguousarray(got[i][:, :n]), want, f"{add}-{mult} product {i}")


def test_batched_empty_batch_and_column_major(oracle):
    import torch
    batch, m, n, k = 3, 64, 64, 32
    rng = np.random.default_rng(3)
    A = rng.random((batch, k, m)).astype(np.float32)                   # slices are column-major m x k matrices
    B = rng.random((batch, n, k)).astype(np.float32)
    dA, dB = torch.from_numpy(A).cuda().transpose(1, 2), torch.from_numpy(B).cuda().transpose(1, 2)
    dD = torch.zeros(batch, n, m, device="cuda").transpose(1, 2)
    inf = float("inf")
    cuasr_amd.srgemm_batched("minimum", "plus", dA, dB, dD, dD, 0.0, inf, inf, 0.0)   # beta = annihilator: C unread
    got = dD.cpu().numpy()
    for i in range(batch):
        want = oracle.srgemm("minimum", "plus", np.asfortranarray(A[i].T), np.asfortranarray(B[i].T),
                             np.zeros((m, n), np.float32, order="F"), 0.0, np.inf, np.inf)
        assert_same_bits(np.ascontiguousarray(got[i]), np.ascontiguousarray(want), f"product {i}")
    cuasr_amd.srgemm_batched("minimum", "plus", dA[:0], dB[:0], dD[:0], dD[:0], 0.0, inf, inf, 0.0)   # nothing to do


@pytest.mark.parametrize("kernel", ["auto", "valu", "direct", "naive"])
def test_many_small_products_in_one_launch(oracle, kernel):
    """1024 products of 64 x 64 x 64: on the tile kernels the product index is part of the grid.  Every
    product against the oracle, operands of the batch at strides larger than a matrix."""
    import torch
    batch, m, n, k = 1024, 64, 64, 64
    rng = np.random.default_rng(5)
    A = rng.random((batch, m + 4, k)).astype(np.float32)                 # row-major slices, 4 rows of padding between them
    B = rng.random((batch, k, n)).astype(np.float32)
    C = rng.random((batch, m, n)).astype(np.float32)
    dA = torch.from_numpy(A).cuda()
    A = A[:, :m, :]
    dB, dC = torch.from_numpy(B).cuda(), torch.from_numpy(C).cuda()
    dD = torch.zeros(batch, m, n, device="cuda")
    cuasr_amd.srgemm_batched("minimum", "plus", dA[:, :m, :], dB, dC, dD, 0.0, 0.0, float("inf"), 0.0, kernel=kernel)
    got = dD.cpu().numpy()
    for i in range(0, batch, 1 if kernel == "auto" else 37):
        want = oracle.srgemm("minimum", "plus", np.ascontiguousarray(A[i]), B[i], C[i], 0.0, 0.0, np.inf)
        assert_same_bits(got[i], want, f"{kernel} product {i}")


def test_batched_column_major_outputs_and_doubles(oracle):
    """Column-major outputs run as the transposed problem: the batch strides of A and B swap with the operands."""
    import torch
    batch, m, n, k = 70, 96, 40, 130
    rng = np.random.default_rng(8)
    A = rng.random((batch, k, m))            # slice i transposed = column-major m x k
    B = rng.random((batch, n, k))            # slice i transposed = column-major k x n
    C = rng.random((batch, n, m))
    dA, dB, dC = (torch.from_numpy(x).cuda().transpose(1, 2) for x in (A, B, C))
    dD = torch.zeros(batch, n, m, dtype=torch.float64, device="cuda").transpose(1, 2)
    cuasr_amd.srgemm_batched("maximum", "plus", dA, dB, dC, dD, 0.0, 0.0, float("-inf"), 0.0)
    got = dD.cpu().numpy()
    for i in range(batch):
        want = oracle.srgemm("maximum", "plus", np.asfortranarray(A[i].T), np.asfortranarray(B[i].T), np.asfortranarray(C[i].T),
                             0.0, 0.0, -np.inf)
        assert_same_bits(np.ascontiguousarray(got[i]), np.ascontiguousarray(want), f"product {i}")


def test_batch_larger_than_one_grid(oracle):
    """More products than the grid's third dimension holds (65535): several launches, same results."""
    import torch
    batch, m, n, k = 65540, 8, 4, 8
    rng = np.random.default_rng(9)
    A = rng.integers(0, 50, (batch, m, k)).astype(np.float32)
    B = rng.integers(0, 50, (batch, k, n)).astype(np.float32)
    dA, dB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    dD = torch.zeros(batch, m, n, device="cuda")
    inf = float("inf")
    cuasr_amd.srgemm_batched("minimum", "plus", dA, dB, dD, dD, 0.0, inf, inf, 0.0)
    want = (A[:, :, :, None] + B[:, None, :, :]).min(axis=2)            # min-plus of every product, exact in fp32
    assert_same_bits(dD.cpu().numpy(), want, "65540 products")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("kernel", ["auto", "mfma"])
def test_plus_times_batch_on_the_matrix_cores(oracle, dtype, kernel):
    """A batch of plus-times products large enough for the matrix cores: the hand-scheduled tiles take the
    product index from the grid.  Small integers, so the sums are exact in any order; row-major products with
    padding rows between them, one B shared by the whole batch, and a column-major batch."""
    import torch
    batch, m, n, k = 12, 512, 384, 160
    rng = np.random.default_rng(23)
    A = rng.integers(-4, 5, (batch, m + 4, k)).astype(dtype)
    B = rng.integers(-4, 5, (k, n)).astype(dtype)
    C = rng.integers(-9, 9, (batch, m, n)).astype(dtype)
    dA = torch.from_numpy(A).cuda()
    dB = torch.from_numpy(B).cuda().unsqueeze(0).expand(batch, k, n)
    dC = torch.from_numpy(C).cuda()
    dD = torch.zeros(batch, m, n, dtype=dA.dtype, device="cuda")
    cuasr_amd.srgemm_batched("plus", "multiplies", dA[:, :m, :], dB, dC, dD, 1.0, 1.0, 0.0, 1.0, kernel=kernel)
    got = dD.cpu().numpy()
    for i in range(batch):
        want = oracle.srgemm("plus", "multiplies", np.ascontiguousarray(A[i, :m]), B, C[i], 1.0, 1.0, 0.0)
        assert_same_bits(got[i], want, f"{kernel} product {i}")
    # column-major products (the transposed problem: A and B swap, and so do their batch strides)
    At = rng.integers(-4, 5, (batch, k, m)).astype(dtype)              # slices are column-major m x k
    Bt = rng.integers(-4, 5, (batch, n, k)).astype(dtype)
    dAt, dBt = torch.from_numpy(At).cuda().transpose(1, 2), torch.from_numpy(Bt).cuda().transpose(1, 2)
    dDt = torch.zeros(batch, n, m, dtype=dAt.dtype, device="cuda").transpose(1, 2)
    cuasr_amd.srgemm_batched("plus", "multiplies", dAt, dBt, dDt, dDt, 1.0, 0.0, 0.0, 1.0, kernel=kernel)
    got = dDt.cpu().numpy()
    for i in range(0, batch, 5):
        want = oracle.srgemm("plus", "multiplies", np.asfortranarray(At[i].T), np.asfortranarray(Bt[i].T),
                             np.zeros((m, n), dtype, order="F"), 1.0, 0.0, 0.0)
        assert_same_bits(np.ascontiguousarray(got[i]), np.ascontiguousarray(want), f"{kernel} column-major product {i}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_batch_strides_off_the_vector_alignment(oracle, dtype):
    """Products whose operands start at odd element offsets (strides of one matrix + 1, + 3 ...): the batch
    stays in the grid but leaves the direct-to-LDS tiles, whose 16-byte loads need every product aligned."""
    import torch
    batch, m, n, k = 64, 512, 512, 96      # 512 direct tiles: with aligned strides this batch takes the direct-to-LDS tile
    rng = np.random.default_rng(23)
    tdt = torch.float32 if dtype == np.float32 else torch.float64

    def strided(rows, cols, extra, lo, hi):
        flat = rng.uniform(lo, hi, batch * (rows * cols + extra)).astype(dtype)
        dev = torch.from_numpy(flat).cuda()
        view = torch.as_strided(dev, (batch, rows, cols), (rows * cols + extra, cols, 1))
        host = np.lib.stride_tricks.as_strided(flat, (batch, rows, cols), ((rows * cols + extra) * flat.itemsize, cols * flat.itemsize, flat.itemsize))
        return dev, view, host

    _, dA, A = strided(m, k, 1, 0, 10)
    _, dB, B = strided(k, n, 3, 0, 10)
    _, dC, C = strided(m, n, 5, 0, 30)
    flatD = torch.full((batch * (m * n + 7),), -5, dtype=tdt, device="cuda")
    dD = torch.as_strided(flatD, (batch, m, n), (m * n + 7, n, 1))
    d = cuasr_amd.make_desc("minimum", "plus", "f32" if dtype == np.float32 else "f64", dA[0], dB[0], dC[0], dD[0], 0.0, 0.0, np.inf, 0.0, 1, "auto")
    import ctypes
    name = cuasr_amd.load().cuasr_amd_selected_kernel_batched(ctypes.byref(d), batch, dA.stride(0), dB.stride(0), dC.stride(0), dD.stride(0))
    assert name == b"valu"
    whole = cuasr_amd.load().cuasr_amd_selected_kernel_batched(ctypes.byref(d), batch, m * k, k * n, m * n, m * n)
    assert whole == b"valu_direct"
    cuasr_amd.srgemm_batched("minimum", "plus", dA, dB, dC, dD, 0.0, 0.0, float("inf"), 0.0)
    got = torch.as_strided(flatD, (batch, m, n), (m * n + 7, n, 1)).cpu().numpy()
    for i in list(range(0, batch, 7)) + [1, batch - 1]:
        want = oracle.srgemm("minimum", "plus", np.ascontiguousarray(A[i]), np.ascontiguousarray(B[i]), np.ascontiguousarray(C[i]), 0.0, 0.0, np.inf)
        assert_same_bits(np.ascontiguousarray(got[i]), want, f"product {i}")
    assert (flatD.cpu().numpy().reshape(batch, m * n + 7)[:, m * n:] == -5).all()      # the gaps between the outputs are untouched
