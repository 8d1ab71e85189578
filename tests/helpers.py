"""Shared helpers of the parity tests: semiring tables, device upload that
keeps the matrix layout, and the bit-exact comparison."""
import numpy as np

NP_OF = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "u32": np.uint32, "f16": np.float16}


def to_device(a):
    """numpy 2-D array (row- or column-major) -> torch CUDA tensor, same layout."""
    import torch
    if a.dtype == np.uint32:
        a = a.view(np.int32)
    if a.flags["C_CONTIGUOUS"]:
        return torch.from_numpy(a).cuda()
    if a.flags["F_CONTIGUOUS"]:
        return torch.from_numpy(np.ascontiguousarray(a.T)).cuda().t()
    raise ValueError("expected a contiguous row- or column-major array")


def to_host(t, dtype):
    a = t.cpu().numpy()
    return a.view(np.uint32) if dtype == "u32" else a


def order_of(layout):
    return "F" if layout == "col" else "C"


def same_bits(x, y):
    x = np.ascontiguousarray(x)
    y = np.ascontiguousarray(y)
    return x.shape == y.shape and x.dtype == y.dtype and x.tobytes() == y.tobytes()


def assert_same_bits(got, want, what=""):
    if same_bits(got, want):
        return
    g = np.ascontiguousarray(got)
    w = np.ascontiguousarray(want)
    ui = {2: np.uint16, 4: np.uint32, 8: np.uint64}[g.itemsize]
    bad = np.argwhere(g.view(ui) != w.view(ui))
    i = tuple(bad[0])
    raise AssertionError(f"{what}: {len(bad)} of {g.size} elements differ; first at {i}: "
                         f"got {g[i]!r} want {w[i]!r}")
