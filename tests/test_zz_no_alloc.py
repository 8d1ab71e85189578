"""cuasr_amd_srgemm_splitk_static: split-K whose partial tiles go to the library's own fixed
device array, for callers that cannot allocate.  It must give cuasr_amd_srgemm_splitk's result
bit for bit (same kernels, only the workspace differs), also on a second, smaller call that
finds the first call's partial tiles still in the array."""
import ctypes

import numpy as np
import pytest

from helpers import assert_same_bits, to_device, to_host

pytestmark = pytest.mark.gpu


def _both(add, mult, dtype, m, n, k, slices, layouts, one, beta, ident, seed, fill):
    """The same problem through the caller-workspace entry point and the static one."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    npd = {"f32": np.float32, "f64": np.float64, "u32": np.uint32}[dtype]
    oa, ob, oc = ("F" if c == "c" else "C" for c in layouts)
    if dtype == "u32":
        A, B, C = inputs.words32(seed, m, k, oa), inputs.words32(seed + 1, k, n, ob), inputs.words32(seed + 2, m, n, oc)
    else:
        A = inputs.uniform(seed, m, k, 0.0, 10.0, npd, oa)
        B = inputs.uniform(seed + 1, k, n, 0.0, 10.0, npd, ob)
        C = inputs.uniform(seed + 2, m, n, 0.0, 10.0, npd, oc)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    ws = torch.empty(cuasr_amd.splitk_workspace_bytes(m, n, slices, dtype), dtype=torch.uint8, device="cuda")
    want = to_device(np.full_like(C, fill))
    got = to_device(np.full_like(C, fill))
    cuasr_amd.srgemm_splitk(add, mult, dA, dB, dC, want, slices, ws, one, beta, ident, one, dtype=dtype)
    cuasr_amd.srgemm_splitk_static(add, mult, dA, dB, dC, got, slices, one, beta, ident, one, dtype=dtype)
    torch.cuda.synchronize()
    return to_host(got, dtype), to_host(want, dtype), (A, B, C)


def test_static_splitk_two_calls_second_smaller(oracle, lib):
    inf = float("inf")
    # first call: 256 x 256 x 8192 in 16 slices (4 MiB of partial tiles); second: a smaller, ragged
    # problem with fewer slices, which finds the first call's partial tiles still in the array
    print("static split-K: 256x256x8192 S=16 min-plus f32", flush=True)
    got, want, (A, B, C) = _both("minimum", "plus", "f32", 256, 256, 8192, 16, "rcr", 0.0, 0.0, inf, 901, 7.0)
    assert_same_bits(got, want, "first call vs cuasr_amd_srgemm_splitk")
    assert_same_bits(got, oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, np.inf), "first call vs oracle")
    print("static split-K: 100x52x1000 S=5 min-plus f32", flush=True)
    got, want, (A, B, C) = _both("minimum", "plus", "f32", 100, 52, 1000, 5, "ccc", 0.0, inf, inf, 911, 7.0)
    assert_same_bits(got, want, "second, smaller call vs cuasr_amd_srgemm_splitk")
    assert_same_bits(got, oracle.srgemm("minimum", "plus", A, B, C, 0.0, inf, np.inf), "second call vs oracle")


def test_static_splitk_other_types(oracle, lib):
    inf = float("inf")
    print("static split-K: 128x192x2048 S=8 max-plus f64", flush=True)
    got, want, (A, B, C) = _both("maximum", "plus", "f64", 128, 192, 2048, 8, "crc", 0.0, 0.0, -inf, 921, 3.0)
    assert_same_bits(got, want, "f64 vs cuasr_amd_srgemm_splitk")
    assert_same_bits(got, oracle.srgemm("maximum", "plus", A, B, C, 0.0, 0.0, -np.inf), "f64 vs oracle")
    print("static split-K: 64x64x4096 S=64 xor-and u32", flush=True)
    got, want, (A, B, C) = _both("bit_xor", "bit_and", "u32", 64, 64, 4096, 64, "ccc", 0xFFFFFFFF, 0xFFFFFFFF, 0, 931, 5)
    assert_same_bits(got, want, "u32 vs cuasr_amd_srgemm_splitk")
    assert_same_bits(got, oracle.srgemm("bit_xor", "bit_and", A, B, C, 0xFFFFFFFF, 0xFFFFFFFF, 0), "u32 vs oracle")


def test_static_splitk_rejects_what_does_not_fit(lib):
    import torch
    import cuasr_amd
    # 1024 x 1024 x 16 slices of f32 = 64 MiB of partial tiles: more than the array holds
    t = torch.zeros(1024, 1024, device="cuda")
    d = cuasr_amd.make_desc("minimum", "plus", "f32", t, t, t, torch.empty_like(t), 0.0, 0.0, float("inf"), 0.0, 16)
    assert lib.cuasr_amd_srgemm_splitk_static(ctypes.byref(d), None) == 10   # kErrorMemoryAllocation
    d.split_k_slices = 4                                                      # 16 MiB: exactly the array
    assert cuasr_amd.splitk_workspace_bytes(1024, 1024, 4, "f32") == cuasr_amd.STATIC_WORKSPACE_BYTES
    assert lib.cuasr_amd_srgemm_splitk_static(ctypes.byref(d), None) == 0
    torch.cuda.synchronize()
