"""CPU oracle for semiring GEMM -- TEST INFRASTRUCTURE ONLY.

Loads ``oracle/liboracle.so`` (built from ``oracle/host_srgemm.c``, a C
restatement of the reference host SRGEMM,
tools/include/cuasr/reference/srgemm/host_srgemm.h:33-113) and exposes it on
numpy arrays.  Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import this package; the shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

OPS = {"plus": 0, "multiplies": 1, "minimum": 2, "maximum": 3, "logical_and": 4,
       "logical_or": 5, "bit_and": 6, "bit_or": 7, "bit_xor": 8}
DTYPES = {np.dtype(np.float32): 0, np.dtype(np.float64): 1,
          np.dtype(np.int32): 2, np.dtype(np.uint32): 3, np.dtype(np.float16): 4}
COLUMN_MAJOR, ROW_MAJOR = 0, 1

_lib = None


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "liboracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_srgemm.restype = ctypes.c_int
        _lib.oracle_srgemm_splitk.restype = ctypes.c_int
        _lib.oracle_srgemm_splitk_serial.restype = ctypes.c_int
        _lib.oracle_max_threads.restype = ctypes.c_int
    return _lib


def max_threads():
    return int(lib().oracle_max_threads())


def mat_ref(a):
    """(pointer, leading dimension, layout) of a 2-D array whose rows or
    columns are contiguous; views with ld > extent are fine."""
    assert a.ndim == 2
    isz = a.itemsize
    s0, s1 = a.strides
    rows, cols = a.shape
    if s0 == isz and (cols <= 1 or (s1 % isz == 0 and s1 // isz >= rows)):
        layout, ld = COLUMN_MAJOR, (s1 // isz if cols > 1 else max(rows, 1))
    elif s1 == isz and (rows <= 1 or (s0 % isz == 0 and s0 // isz >= cols)):
        layout, ld = ROW_MAJOR, (s0 // isz if rows > 1 else max(cols, 1))
    elif rows == 1 and cols == 1:
        layout, ld = COLUMN_MAJOR, 1
    else:
        raise ValueError("matrix must have unit stride along rows or columns")
    return a.ctypes.data_as(ctypes.c_void_p), int(ld), layout


def _element_types(A, B, C):
    """(dtype of C, D and the scalars; the oracle's type code).  int8 operands go with int32 everything else."""
    if A.dtype == np.int8:
        assert B.dtype == np.int8 and C.dtype == np.int32
        return np.dtype(np.int32), 5
    assert B.dtype == A.dtype and C.dtype == A.dtype
    return A.dtype, DTYPES[A.dtype]


def _scalar(v, dtype):
    return np.array([v], dtype=dtype)


def empty_like_layout(c, shape=None):
    """New array with the same layout (row/column major) as ``c``."""
    _, _, layout = mat_ref(c)
    shape = shape or c.shape
    return np.empty(shape, dtype=c.dtype, order="F" if layout == COLUMN_MAJOR else "C")


def srgemm(add_op, mult_op, A, B, C, alpha, beta, add_identity, out=None,
           nthreads=0, naive=False):
    """D = add(mult(alpha, A (x) B), mult(beta, C)) on the CPU oracle.

    A is m x k, B is k x n, C is m x n; each row- or column-major (taken from
    the strides).  D gets C's layout.  Returns D.
    """
    dt, code = _element_types(A, B, C)
    m, k = A.shape
    k2, n = B.shape
    assert k2 == k and C.shape == (m, n)
    D = out if out is not None else empty_like_layout(C)
    pa, lda, la = mat_ref(A)
    pb, ldb, lb = mat_ref(B)
    pc, ldc, lc = mat_ref(C)
    pd, ldd, ld_layout = mat_ref(D)
    assert ld_layout == lc or m == 1 or n == 1
    al, be, ident = _scalar(alpha, dt), _scalar(beta, dt), _scalar(add_identity, dt)
    rc = lib().oracle_srgemm(
        code, OPS[add_op], OPS[mult_op], m, n, k,
        al.ctypes.data_as(ctypes.c_void_p), pa, ctypes.c_int64(lda), la,
        pb, ctypes.c_int64(ldb), lb, be.ctypes.data_as(ctypes.c_void_p),
        pc, ctypes.c_int64(ldc), pd, ctypes.c_int64(ldd), lc,
        ident.ctypes.data_as(ctypes.c_void_p), int(nthreads), int(bool(naive)))
    if rc != 0:
        raise ValueError(f"oracle: unsupported ({dt}, {add_op}, {mult_op})")
    return D


def srgemm_splitk(add_op, mult_op, A, B, C, alpha, beta, add_identity,
                  mult_identity, slices, tbk=8, out=None, nthreads=0):
    """CPU model of the two-kernel parallel split-K (partials, then reduce)."""
    dt, code = _element_types(A, B, C)
    m, k = A.shape
    _, n = B.shape
    D = out if out is not None else empty_like_layout(C)
    pa, lda, la = mat_ref(A)
    pb, ldb, lb = mat_ref(B)
    pc, ldc, lc = mat_ref(C)
    pd, ldd, _ = mat_ref(D)
    al, be = _scalar(alpha, dt), _scalar(beta, dt)
    ident, one = _scalar(add_identity, dt), _scalar(mult_identity, dt)
    rc = lib().oracle_srgemm_splitk(
        code, OPS[add_op], OPS[mult_op], m, n, k,
        al.ctypes.data_as(ctypes.c_void_p), pa, ctypes.c_int64(lda), la,
        pb, ctypes.c_int64(ldb), lb, be.ctypes.data_as(ctypes.c_void_p),
        pc, ctypes.c_int64(ldc), pd, ctypes.c_int64(ldd), lc,
        ident.ctypes.data_as(ctypes.c_void_p), one.ctypes.data_as(ctypes.c_void_p),
        int(slices), int(tbk), int(nthreads))
    if rc != 0:
        raise ValueError(f"oracle: unsupported split-K ({dt}, {add_op}, {mult_op})")
    return D


def srgemm_splitk_serial(add_op, mult_op, A, B, C, alpha, beta, add_identity,
                         mult_identity, slices, tbk=8, out=None, nthreads=0):
    """CPU model of the serial split-K: the slices' epilogues chained through D."""
    dt, code = _element_types(A, B, C)
    m, k = A.shape
    _, n = B.shape
    D = out if out is not None else empty_like_layout(C)
    pa, lda, la = mat_ref(A)
    pb, ldb, lb = mat_ref(B)
    pc, ldc, lc = mat_ref(C)
    pd, ldd, _ = mat_ref(D)
    al, be = _scalar(alpha, dt), _scalar(beta, dt)
    ident, one = _scalar(add_identity, dt), _scalar(mult_identity, dt)
    rc = lib().oracle_srgemm_splitk_serial(
        code, OPS[add_op], OPS[mult_op], m, n, k,
        al.ctypes.data_as(ctypes.c_void_p), pa, ctypes.c_int64(lda), la,
        pb, ctypes.c_int64(ldb), lb, be.ctypes.data_as(ctypes.c_void_p),
        pc, ctypes.c_int64(ldc), pd, ctypes.c_int64(ldd), lc,
        ident.ctypes.data_as(ctypes.c_void_p), one.ctypes.data_as(ctypes.c_void_p),
        int(slices), int(tbk), int(nthreads))
    if rc != 0:
        raise ValueError(f"oracle: unsupported serial split-K ({dt}, {add_op}, {mult_op})")
    return D


def fwgemm(A, B, dist, parent, nthreads=0):
    """Min-plus product with predecessor tracking, in place on ``dist`` and
    ``parent`` (column-major float32/float64 and int32 arrays), following
    test/regress/include/fwgpu/cpu_srgemm.hpp:20-48."""
    dt = A.dtype
    m, k = A.shape
    _, n = B.shape
    if m == 0 or n == 0 or k == 0:
        return dist, parent          # an empty scan changes nothing
    refs = [mat_ref(x) for x in (A, B, dist, parent)]
    if any(r[2] != COLUMN_MAJOR for r in refs) or parent.dtype != np.int32 or dist.shape != (m, n):
        raise ValueError("oracle.fwgemm: column-major operands and an int32 parent matrix")
    (pa, lda, _), (pb, ldb, _), (pd, ldc, _), (pp, ldp, _) = refs
    fn = lib().oracle_fwgemm
    fn.restype = ctypes.c_int
    rc = fn(DTYPES[dt], m, n, k, pa, ctypes.c_int64(lda), pb, ctypes.c_int64(ldb),
            pd, ctypes.c_int64(ldc), pp, ctypes.c_int64(ldp), int(nthreads))
    if rc != 0:
        raise ValueError(f"oracle.fwgemm: unsupported element type {dt}")
    return dist, parent


def apsp_blocked(dist, parent, block=128):
    """Blocked Floyd-Warshall with predecessor tracking, in place on a square
    column-major ``dist`` (float32/float64) and an int32 ``parent``; the order of
    operations is the device driver's (see host_blocked_fw.c)."""
    n = dist.shape[0]
    if n == 0:
        return dist, parent
    refs = [mat_ref(x) for x in (dist, parent)]
    if any(r[2] != COLUMN_MAJOR for r in refs) or parent.dtype != np.int32 or dist.shape != (n, n) or parent.shape != (n, n):
        raise ValueError("oracle.apsp_blocked: square column-major dist and an int32 parent matrix")
    (pd, ld, _), (pp, ldp, _) = refs
    fn = lib().oracle_apsp_blocked
    fn.restype = ctypes.c_int
    rc = fn(DTYPES[dist.dtype], n, pd, ctypes.c_int64(ld), pp, ctypes.c_int64(ldp), int(block))
    if rc != 0:
        raise ValueError(f"oracle.apsp_blocked: failed ({rc})")
    return dist, parent
