"""cuasr_amd: semiring GEMM for AMD Instinct MI355X (gfx950).

The product is ``lib/libcuasr_amd.so`` (hand-written HIP kernels behind the C
ABI of ``include/cuasr_amd.h``) and the C++ operator templates in
``include/cuasr/`` that mirror cuASR's ``device::Srgemm`` /
``device::SrgemmSplitKParallel``.  This module is a thin ctypes binding of the
same C ABI for Python callers (tests, the benchmark); torch tensors are used
only as handles to device memory.  There is no CPU fallback: if the library
has not been built, loading raises.
"""
import ctypes
import struct
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("CUASR_AMD_LIB") or os.path.join(_HERE, "lib", "libcuasr_amd.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "cuasr_amd.h")

# enums of include/cuasr_amd.h
OPS = {"plus": 0, "multiplies": 1, "minimum": 2, "maximum": 3, "logical_and": 4,
       "logical_or": 5, "bit_and": 6, "bit_or": 7, "bit_xor": 8}
DTYPES = {"f32": 0, "f64": 1, "i32": 2, "u32": 3, "f16": 4, "i8": 5}
COLUMN_MAJOR, ROW_MAJOR = 0, 1
KERNELS = {"auto": 0, "naive": 1, "valu": 2, "mfma": 3, "direct": 4, "streamk": 5}
STATUS_NAMES = ["kSuccess", "kErrorMisalignedOperand", "kErrorInvalidDataType",
                "kErrorInvalidLayout", "kErrorInvalidProblem", "kErrorNotSupported",
                "kErrorWorkspaceNull", "kErrorInternal", "kErrorArchMismatch",
                "kErrorInsufficientDriver", "kErrorMemoryAllocation", "kInvalid"]
SUCCESS = 0

_NP_OF = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "u32": np.uint32, "f16": np.float16,
          "i8": np.int32}   # (int8 operands: the scalars, C and D are int32)


class Scalar(ctypes.Union):
    _fields_ = [("f32", ctypes.c_float), ("f64", ctypes.c_double), ("i32", ctypes.c_int32),
                ("u32", ctypes.c_uint32), ("f16", ctypes.c_uint16), ("bits", ctypes.c_uint64)]


class SrgemmDesc(ctypes.Structure):
    """cuasr_amd_srgemm_desc"""
    _fields_ = [
        ("add_op", ctypes.c_int32), ("mult_op", ctypes.c_int32), ("dtype", ctypes.c_int32),
        ("layout_a", ctypes.c_int32), ("layout_b", ctypes.c_int32), ("layout_c", ctypes.c_int32),
        ("m", ctypes.c_int32), ("n", ctypes.c_int32), ("k", ctypes.c_int32),
        ("split_k_slices", ctypes.c_int32),
        ("A", ctypes.c_void_p), ("lda", ctypes.c_int64),
        ("B", ctypes.c_void_p), ("ldb", ctypes.c_int64),
        ("C", ctypes.c_void_p), ("ldc", ctypes.c_int64),
        ("D", ctypes.c_void_p), ("ldd", ctypes.c_int64),
        ("alpha", Scalar), ("beta", Scalar), ("add_identity", Scalar), ("mult_identity", Scalar),
        ("alpha_ptr", ctypes.c_void_p), ("beta_ptr", ctypes.c_void_p),
        ("kernel", ctypes.c_int32), ("reserved", ctypes.c_int32),
    ]


class CuasrError(RuntimeError):
    def __init__(self, status, what):
        self.status = int(status)
        name = STATUS_NAMES[self.status] if 0 <= self.status < len(STATUS_NAMES) else "?"
        super().__init__(f"{what}: status {self.status} ({name})")


_lib = None


def load():
    """Load the built library; raises if it is missing (no fallback)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is not built; run `python -m cuasr_amd.build` (needs hipcc). "
                "cuasr_amd has no CPU fallback.")
        lib = ctypes.CDLL(LIB_PATH)
        lib.cuasr_amd_abi_version.restype = ctypes.c_int
        lib.cuasr_amd_status_string.restype = ctypes.c_char_p
        lib.cuasr_amd_status_string.argtypes = [ctypes.c_int]
        lib.cuasr_amd_srgemm_can_implement.restype = ctypes.c_int
        lib.cuasr_amd_srgemm_can_implement.argtypes = [ctypes.POINTER(SrgemmDesc)]
        lib.cuasr_amd_srgemm.restype = ctypes.c_int
        lib.cuasr_amd_srgemm.argtypes = [ctypes.POINTER(SrgemmDesc), ctypes.c_void_p]
        lib.cuasr_amd_srgemm_batched.restype = ctypes.c_int
        lib.cuasr_amd_srgemm_batched.argtypes = [ctypes.POINTER(SrgemmDesc), ctypes.c_int] + [ctypes.c_int64] * 4 + [ctypes.c_void_p]
        lib.cuasr_amd_splitk_workspace_bytes.restype = ctypes.c_size_t
        lib.cuasr_amd_splitk_workspace_bytes.argtypes = [ctypes.POINTER(SrgemmDesc)]
        lib.cuasr_amd_srgemm_splitk.restype = ctypes.c_int
        lib.cuasr_amd_srgemm_splitk.argtypes = [ctypes.POINTER(SrgemmDesc), ctypes.c_void_p, ctypes.c_void_p]
        lib.cuasr_amd_reduce_splitk.restype = ctypes.c_int
        lib.cuasr_amd_reduce_splitk.argtypes = [ctypes.POINTER(SrgemmDesc), ctypes.c_void_p, ctypes.c_void_p]
        lib.cuasr_amd_srgemm_splitk_static.restype = ctypes.c_int
        lib.cuasr_amd_srgemm_splitk_static.argtypes = [ctypes.POINTER(SrgemmDesc), ctypes.c_void_p]
        lib.cuasr_amd_splitk_serial_workspace_bytes.restype = ctypes.c_size_t
        lib.cuasr_amd_splitk_serial_workspace_bytes.argtypes = [ctypes.POINTER(SrgemmDesc)]
        lib.cuasr_amd_srgemm_splitk_serial.restype = ctypes.c_int
        lib.cuasr_amd_srgemm_splitk_serial.argtypes = [ctypes.POINTER(SrgemmDesc), ctypes.c_void_p, ctypes.c_void_p]
        lib.cuasr_amd_fwgemm.restype = ctypes.c_int
        lib.cuasr_amd_fwgemm.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_int64] * 4 + [ctypes.c_int, ctypes.c_void_p]
        lib.cuasr_amd_apsp_workspace_bytes.restype = ctypes.c_size_t
        lib.cuasr_amd_apsp_workspace_bytes.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.cuasr_amd_apsp_blocked_workspace_bytes.restype = ctypes.c_size_t
        lib.cuasr_amd_apsp_blocked_workspace_bytes.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.cuasr_amd_apsp_blocked.restype = ctypes.c_int
        lib.cuasr_amd_apsp_blocked.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                               ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
        lib.cuasr_amd_apsp_blocked_panels.restype = ctypes.c_int
        lib.cuasr_amd_apsp_blocked_panels.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                                      ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        lib.cuasr_amd_apsp_squaring.restype = ctypes.c_int
        lib.cuasr_amd_apsp_squaring.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                                ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
        lib.cuasr_amd_selected_kernel.restype = ctypes.c_char_p
        lib.cuasr_amd_selected_kernel.argtypes = [ctypes.POINTER(SrgemmDesc)]
        lib.cuasr_amd_selected_kernel_batched.restype = ctypes.c_char_p
        lib.cuasr_amd_selected_kernel_batched.argtypes = [ctypes.POINTER(SrgemmDesc), ctypes.c_int] + [ctypes.c_int64] * 4
        _lib = lib
    return _lib


# --------------------------------------------------------------------------
# Semiring constants, as the reference functors define them
# (include/cuasr/functional.h:28-36, :41-42, :84-85, :127-128, :167-168,
#  :207-208, :247-248; binary_xor: examples/01_userdefined_semiring/
#  userdefined_semiring.cu:57).  "Infinity" there is numeric_limits::max() and
# "-infinity" numeric_limits::min() (the smallest positive normal for floating
# point).  With infinities=True the floating-point values become true +/-inf.
# --------------------------------------------------------------------------
def _limits(dtype, infinities):
    npd = np.dtype(_NP_OF[dtype])
    if npd.kind == "f":
        if infinities:
            return npd.type(np.inf), npd.type(-np.inf)
        fi = np.finfo(npd)
        return fi.max, fi.tiny
    ii = np.iinfo(npd)
    return npd.type(ii.max), npd.type(ii.min)


def op_identity(op, dtype, infinities=False):
    hi, lo = _limits(dtype, infinities)
    npd = _NP_OF[dtype]
    return {"plus": npd(0), "multiplies": npd(1), "minimum": hi, "maximum": lo,
            "logical_and": npd(1), "logical_or": npd(0),
            "bit_and": npd(np.iinfo(npd).max if np.dtype(npd).kind == "u" else -1)
            if np.dtype(npd).kind in "iu" else npd(1),
            "bit_or": npd(0), "bit_xor": npd(0)}[op]


def op_annihilator(op, dtype, infinities=False):
    hi, lo = _limits(dtype, infinities)
    npd = _NP_OF[dtype]
    return {"plus": hi, "multiplies": npd(0), "minimum": lo, "maximum": hi,
            "logical_and": npd(0), "logical_or": npd(1), "bit_and": npd(0),
            "bit_or": npd(np.iinfo(npd).max if np.dtype(npd).kind == "u" else -1)
            if np.dtype(npd).kind in "iu" else npd(1),
            "bit_xor": npd(0)}[op]


def _set_scalar(s, value, dtype):
    s.bits = 0
    if dtype == "f32":
        s.f32 = float(value)
    elif dtype == "f64":
        s.f64 = float(value)
    elif dtype in ("i32", "i8"):
        s.i32 = int(value)
    elif dtype == "f16":
        try:                                                   # the binary16 bit pattern, rounded to nearest-even
            s.f16 = struct.unpack("<H", struct.pack("<e", float(value)))[0]
        except OverflowError:                                  # beyond 65504: struct refuses, numpy rounds to infinity
            s.f16 = int(np.array([value], dtype=np.float16).view(np.uint16)[0])
    else:
        s.u32 = int(value) & 0xFFFFFFFF


class MatRef:
    """A matrix in device memory: pointer, leading dimension (elements), layout."""

    def __init__(self, ptr, ld, layout, rows, cols):
        self.ptr, self.ld, self.layout, self.rows, self.cols = int(ptr or 0), int(ld), int(layout), int(rows), int(cols)

    @staticmethod
    def of(t):
        """From a 2-D torch tensor whose rows or columns are contiguous."""
        if isinstance(t, MatRef):
            return t
        rows, cols = t.shape
        s0, s1 = t.stride()
        if s0 == 1 and (cols <= 1 or s1 >= rows):
            return MatRef(t.data_ptr(), s1 if cols > 1 else max(rows, 1), COLUMN_MAJOR, rows, cols)
        if s1 == 1 and (rows <= 1 or s0 >= cols):
            return MatRef(t.data_ptr(), s0 if rows > 1 else max(cols, 1), ROW_MAJOR, rows, cols)
        raise ValueError("matrix must have unit stride along rows or columns")


def _torch_dtype_name(t):
    import torch
    return {torch.float32: "f32", torch.float64: "f64", torch.int32: "i32",
            getattr(torch, "uint32", None): "u32", torch.float16: "f16"}[t.dtype]


def make_desc(add_op, mult_op, dtype, A, B, C, D, alpha, beta, add_identity, mult_identity,
              split_k_slices=1, kernel="auto", alpha_ptr=None, beta_ptr=None):
    a, b, d = MatRef.of(A), MatRef.of(B), MatRef.of(D)
    c = MatRef.of(C) if C is not None else MatRef(0, d.ld, d.layout, d.rows, d.cols)
    desc = SrgemmDesc()
    desc.add_op, desc.mult_op, desc.dtype = OPS[add_op], OPS[mult_op], DTYPES[dtype]
    desc.layout_a, desc.layout_b, desc.layout_c = a.layout, b.layout, d.layout
    if c.ptr and c.layout != d.layout:
        # only a contiguous vector can be read in either layout
        if min(d.rows, d.cols) > 1 or c.ld != (1 if (c.layout == COLUMN_MAJOR) == (c.rows == 1) else max(c.rows, c.cols)):
            raise ValueError("C and D must share a layout")
        c = MatRef(c.ptr, max(c.cols, 1) if d.layout == ROW_MAJOR and c.rows == 1 else
                   max(c.rows, 1) if d.layout == COLUMN_MAJOR and c.cols == 1 else 1, d.layout, c.rows, c.cols)
    if a.cols != b.rows or (a.rows, b.cols) != (d.rows, d.cols):
        raise ValueError("shape mismatch")
    desc.m, desc.n, desc.k = d.rows, d.cols, a.cols
    desc.split_k_slices = split_k_slices
    desc.A, desc.lda = a.ptr or None, a.ld
    desc.B, desc.ldb = b.ptr or None, b.ld
    desc.C, desc.ldc = c.ptr or None, c.ld
    desc.D, desc.ldd = d.ptr or None, d.ld
    _set_scalar(desc.alpha, alpha, dtype)
    _set_scalar(desc.beta, beta, dtype)
    _set_scalar(desc.add_identity, add_identity, dtype)
    _set_scalar(desc.mult_identity, mult_identity, dtype)
    desc.alpha_ptr = alpha_ptr
    desc.beta_ptr = beta_ptr
    desc.kernel = KERNELS[kernel]
    desc.reserved = 0
    return desc


def _stream_handle(stream):
    if stream is None:
        import torch
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return ctypes.c_void_p(int(getattr(stream, "cuda_stream", stream)))


def srgemm(add_op, mult_op, A, B, C, D, alpha=None, beta=None, add_identity=None,
           mult_identity=None, dtype=None, kernel="auto", stream=None,
           alpha_ptr=None, beta_ptr=None, infinities=False):
    """D = add(mult(alpha, A (x) B), mult(beta, C)) on the GPU, asynchronously.

    Defaults follow the reference epilogue (semiring_linear_combination.h:67-71):
    alpha = MultOp::Identity, beta = MultOp::Annihilator; the identities default
    to the reference functor constants (or +/-inf with ``infinities=True``).
    """
    dtype = dtype or _torch_dtype_name(D)
    alpha = op_identity(mult_op, dtype, infinities) if alpha is None else alpha
    beta = op_annihilator(mult_op, dtype, infinities) if beta is None else beta
    add_identity = op_identity(add_op, dtype, infinities) if add_identity is None else add_identity
    mult_identity = op_identity(mult_op, dtype, infinities) if mult_identity is None else mult_identity
    desc = make_desc(add_op, mult_op, dtype, A, B, C, D, alpha, beta, add_identity, mult_identity,
                     1, kernel, alpha_ptr, beta_ptr)
    st = load().cuasr_amd_srgemm(ctypes.byref(desc), _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_srgemm")
    return D


def srgemm_batched(add_op, mult_op, A, B, C, D, alpha, beta, add_identity, mult_identity, dtype=None,
                   kernel="auto", stream=None):
    """A batch of SRGEMMs: A, B, C, D are 3-D CUDA tensors (batch, rows, cols) whose 2-D slices are
    row- or column-major matrices; a first dimension of stride 0 (``expand``) shares an operand."""
    dtype = dtype or _torch_dtype_name(D)
    batch = D.shape[0]
    if batch == 0:
        return D
    desc = make_desc(add_op, mult_op, dtype, A[0], B[0], C[0], D[0], alpha, beta, add_identity, mult_identity, 1, kernel)
    st = load().cuasr_amd_srgemm_batched(ctypes.byref(desc), batch, A.stride(0), B.stride(0), C.stride(0), D.stride(0),
                                         _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_srgemm_batched")
    return D


def splitk_workspace_bytes(m, n, slices, dtype):
    desc = SrgemmDesc()
    desc.m, desc.n, desc.split_k_slices, desc.dtype = m, n, slices, DTYPES[dtype]
    return int(load().cuasr_amd_splitk_workspace_bytes(ctypes.byref(desc)))


def srgemm_splitk(add_op, mult_op, A, B, C, D, slices, workspace, alpha=None, beta=None,
                  add_identity=None, mult_identity=None, dtype=None, kernel="auto",
                  stream=None, alpha_ptr=None, beta_ptr=None, infinities=False):
    """Parallel split-K SRGEMM: partial products of ``slices`` K-slices into
    ``workspace`` (device memory, >= splitk_workspace_bytes), then a reduction
    with the semiring's add and the epilogue."""
    dtype = dtype or _torch_dtype_name(D)
    alpha = op_identity(mult_op, dtype, infinities) if alpha is None else alpha
    beta = op_annihilator(mult_op, dtype, infinities) if beta is None else beta
    add_identity = op_identity(add_op, dtype, infinities) if add_identity is None else add_identity
    mult_identity = op_identity(mult_op, dtype, infinities) if mult_identity is None else mult_identity
    desc = make_desc(add_op, mult_op, dtype, A, B, C, D, alpha, beta, add_identity, mult_identity,
                     slices, kernel, alpha_ptr, beta_ptr)
    ws = workspace.data_ptr() if hasattr(workspace, "data_ptr") else workspace
    st = load().cuasr_amd_srgemm_splitk(ctypes.byref(desc), ctypes.c_void_p(ws or None), _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_srgemm_splitk")
    return D


STATIC_WORKSPACE_BYTES = 16 << 20  # CUASR_AMD_STATIC_WORKSPACE_BYTES


def srgemm_splitk_static(add_op, mult_op, A, B, C, D, slices, alpha=None, beta=None,
                         add_identity=None, mult_identity=None, dtype=None, kernel="auto",
                         stream=None, alpha_ptr=None, beta_ptr=None, infinities=False):
    """Parallel split-K SRGEMM whose partial tiles go to the library's own fixed device array
    (STATIC_WORKSPACE_BYTES per GPU) instead of a caller workspace: the call allocates nothing.
    Calls that may overlap on one GPU share that array and must be ordered by the caller."""
    dtype = dtype or _torch_dtype_name(D)
    alpha = op_identity(mult_op, dtype, infinities) if alpha is None else alpha
    beta = op_annihilator(mult_op, dtype, infinities) if beta is None else beta
    add_identity = op_identity(add_op, dtype, infinities) if add_identity is None else add_identity
    mult_identity = op_identity(mult_op, dtype, infinities) if mult_identity is None else mult_identity
    desc = make_desc(add_op, mult_op, dtype, A, B, C, D, alpha, beta, add_identity, mult_identity,
                     slices, kernel, alpha_ptr, beta_ptr)
    st = load().cuasr_amd_srgemm_splitk_static(ctypes.byref(desc), _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_srgemm_splitk_static")
    return D


def splitk_serial_workspace_bytes(m, n, slices, dtype):
    desc = SrgemmDesc()
    desc.m, desc.n, desc.split_k_slices, desc.dtype = m, n, slices, DTYPES[dtype]
    return int(load().cuasr_amd_splitk_serial_workspace_bytes(ctypes.byref(desc)))


def srgemm_splitk_serial(add_op, mult_op, A, B, C, D, slices, workspace, alpha=None, beta=None,
                         add_identity=None, mult_identity=None, dtype=None, kernel="auto",
                         stream=None, alpha_ptr=None, beta_ptr=None, infinities=False):
    """Serial split-K SRGEMM (the reference's ``SplitKSerial = true``): the result is the chain
    D_0 = add(mult(alpha, acc_0), mult(beta, C)), D_z = add(mult(alpha, acc_z), mult(one, D_{z-1})).
    ``workspace``: device memory of >= splitk_serial_workspace_bytes (None when slices == 1)."""
    dtype = dtype or _torch_dtype_name(D)
    alpha = op_identity(mult_op, dtype, infinities) if alpha is None else alpha
    beta = op_annihilator(mult_op, dtype, infinities) if beta is None else beta
    add_identity = op_identity(add_op, dtype, infinities) if add_identity is None else add_identity
    mult_identity = op_identity(mult_op, dtype, infinities) if mult_identity is None else mult_identity
    desc = make_desc(add_op, mult_op, dtype, A, B, C, D, alpha, beta, add_identity, mult_identity,
                     slices, kernel, alpha_ptr, beta_ptr)
    ws = workspace.data_ptr() if hasattr(workspace, "data_ptr") else workspace
    st = load().cuasr_amd_srgemm_splitk_serial(ctypes.byref(desc), ctypes.c_void_p(ws or None),
                                               _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_srgemm_splitk_serial")
    return D


def _column_major(t, what):
    """(pointer, leading dimension) of a column-major 2-D device tensor."""
    ref = MatRef.of(t)
    if ref.layout != COLUMN_MAJOR:
        raise ValueError(f"{what} must be column-major")
    return ctypes.c_void_p(ref.ptr), ctypes.c_int64(ref.ld)


def fwgemm(A, B, dist, parent, kernel="auto", stream=None):
    """dist = min(dist, A (x) B) with parent[i, j] = the k that gave each new
    minimum, in place (test/regress/include/fwgpu/cpu_srgemm.hpp:20-48).  All
    four are column-major device tensors; parent is int32."""
    import torch
    if parent.dtype != torch.int32:
        raise ValueError("parent must be int32")
    (m, k), n = A.shape, B.shape[1]
    pa, lda = _column_major(A, "A")
    pb, ldb = _column_major(B, "B")
    pd, ldc = _column_major(dist, "dist")
    pp, ldp = _column_major(parent, "parent")
    st = load().cuasr_amd_fwgemm(DTYPES[_torch_dtype_name(dist)], m, n, k, pa, lda, pb, ldb, pd, ldc, pp, ldp,
                                 KERNELS[kernel], _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_fwgemm")
    return dist, parent


def apsp_workspace_bytes(n, dtype):
    return int(load().cuasr_amd_apsp_workspace_bytes(DTYPES[dtype], n))


def apsp_squaring(dist, parent, workspace, iterations=0, stream=None):
    """All-pairs shortest paths by repeated squaring, in place on the n x n
    column-major ``dist`` and int32 ``parent``; ``workspace`` is a device tensor
    of at least apsp_workspace_bytes(n, dtype) bytes."""
    n = dist.shape[0]
    pd, ld = _column_major(dist, "dist")
    pp, ldp = _column_major(parent, "parent")
    ws = ctypes.c_void_p(workspace.data_ptr()) if workspace is not None else None
    st = load().cuasr_amd_apsp_squaring(DTYPES[_torch_dtype_name(dist)], n, pd, ld, pp, ldp, ws, int(iterations),
                                        _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_apsp_squaring")
    return dist, parent


def apsp_blocked_workspace_bytes(n, dtype):
    return int(load().cuasr_amd_apsp_blocked_workspace_bytes(DTYPES[dtype], n))


PANELS = {"auto": 0, "paired": 1, "tiled": 2}


def apsp_blocked(dist, parent, workspace, stream=None, panels="auto"):
    """All-pairs shortest paths by blocked Floyd-Warshall with predecessor
    tracking, in place on the n x n column-major ``dist`` and int32 ``parent``;
    ``workspace`` is a device tensor of at least
    apsp_blocked_workspace_bytes(n, dtype) bytes."""
    n = dist.shape[0]
    pd, ld = _column_major(dist, "dist")
    pp, ldp = _column_major(parent, "parent")
    ws = ctypes.c_void_p(workspace.data_ptr()) if workspace is not None else None
    if panels == "auto":
        st = load().cuasr_amd_apsp_blocked(DTYPES[_torch_dtype_name(dist)], n, pd, ld, pp, ldp, ws, _stream_handle(stream))
    else:
        st = load().cuasr_amd_apsp_blocked_panels(DTYPES[_torch_dtype_name(dist)], n, pd, ld, pp, ldp, ws, PANELS[panels],
                                                  _stream_handle(stream))
    if st != SUCCESS:
        raise CuasrError(st, "cuasr_amd_apsp_blocked")
    return dist, parent
