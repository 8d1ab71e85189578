"""Host-side checks of the C ABI that need no GPU: the library loads, exports
every function include/cuasr_amd.h declares, and validates descriptors like the
reference's can_implement / initialize do."""
import ctypes
import os
import re

import numpy as np
import pytest

import cuasr_amd
from cuasr_amd import COLUMN_MAJOR, ROW_MAJOR, MatRef


def declared_functions():
    text = open(cuasr_amd.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cuasr_amd_[a-z_]+)\s*\(", text)))


def test_exports_match_header(lib):
    names = declared_functions()
    assert {"cuasr_amd_srgemm", "cuasr_amd_srgemm_splitk", "cuasr_amd_splitk_workspace_bytes",
            "cuasr_amd_srgemm_can_implement", "cuasr_amd_srgemm_splitk_serial",
            "cuasr_amd_splitk_serial_workspace_bytes", "cuasr_amd_fwgemm", "cuasr_amd_apsp_squaring",
            "cuasr_amd_apsp_workspace_bytes", "cuasr_amd_apsp_blocked", "cuasr_amd_apsp_blocked_workspace_bytes",
            "cuasr_amd_srgemm_batched", "cuasr_amd_srgemm_splitk_static", "cuasr_amd_reduce_splitk"} <= set(names)
    for name in names:
        assert hasattr(lib, name), name
    assert lib.cuasr_amd_abi_version() == 1


def test_status_strings(lib):
    assert lib.cuasr_amd_status_string(0) == b"success"
    assert lib.cuasr_amd_status_string(6) == b"workspace is null"
    assert len(cuasr_amd.STATUS_NAMES) == 12 and cuasr_amd.STATUS_NAMES[4] == "kErrorInvalidProblem"


def desc(m=64, n=64, k=64, dtype="f32", add="minimum", mult="plus", la=COLUMN_MAJOR, lb=COLUMN_MAJOR, lc=COLUMN_MAJOR,
         ptr=0x10000, **kw):
    A = MatRef(ptr, kw.pop("lda", m if la == COLUMN_MAJOR else k), la, m, k)
    B = MatRef(ptr, kw.pop("ldb", k if lb == COLUMN_MAJOR else n), lb, k, n)
    ldc = kw.pop("ldc", m if lc == COLUMN_MAJOR else n)
    C = MatRef(ptr, ldc, lc, m, n)
    D = MatRef(kw.pop("dptr", ptr), kw.pop("ldd", ldc), lc, m, n)
    return cuasr_amd.make_desc(add, mult, dtype, A, B, C, D, 0, 0, 0, 0, kw.pop("slices", 1), kw.pop("kernel", "auto"))


def test_can_implement(lib):
    ok = lambda d: lib.cuasr_amd_srgemm_can_implement(ctypes.byref(d))
    assert ok(desc()) == 0
    assert ok(desc(slices=2)) == 4            # kErrorInvalidProblem: split-K on the plain operator (device/srgemm.h:198-200)
    assert ok(desc(lda=10)) == 4              # leading dimension smaller than the extent
    assert ok(desc(ptr=0x10002)) == 1         # kErrorMisalignedOperand (kernel/srgemm.h:129-150)
    assert ok(desc(dtype="f64", ptr=0x10004)) == 1
    assert ok(desc(add="bit_xor", mult="bit_and")) == 5            # bitwise on floating point
    assert ok(desc(dtype="u32", add="bit_xor", mult="bit_and")) == 0
    assert ok(desc(dtype="f64", kernel="mfma")) == 5               # no matrix-core tile for this type
    assert ok(desc(kernel="mfma")) == 0
    assert ok(desc(m=63, kernel="mfma")) == 5                      # needs vector-sized contiguous extents
    assert ok(desc(add="plus", mult="bit_or", dtype="i32", kernel="valu")) == 5
    assert ok(desc(add="plus", mult="bit_or", dtype="i32", kernel="naive")) == 0
    d = desc()
    d.dtype = 9
    assert ok(d) == 2
    d = desc()
    d.layout_b = 7
    assert ok(d) == 3
    d = desc()
    d.m = -1
    assert ok(d) == 4
    d = desc(dptr=0)
    assert ok(d) == 4


def test_half_and_int8_element_types(lib):
    ok = lambda d: lib.cuasr_amd_srgemm_can_implement(ctypes.byref(d))
    sel = lambda d: lib.cuasr_amd_selected_kernel(ctypes.byref(d))
    # binary16: two-byte alignment everywhere, no bitwise operators, the packed tile for the tropical pairs and plus-times
    assert ok(desc(dtype="f16", ptr=0x10002)) == 0
    assert ok(desc(dtype="f16", ptr=0x10001)) == 1
    assert ok(desc(dtype="f16", add="bit_xor", mult="bit_and")) == 5
    assert ok(desc(dtype="f16", kernel="mfma")) == 5 and ok(desc(dtype="f16", kernel="direct")) == 5
    assert sel(desc(dtype="f16")) == b"valu" and sel(desc(dtype="f16", m=63, n=1, k=5)) == b"valu"
    assert sel(desc(dtype="f16", add="plus", mult="multiplies")) == b"valu"
    # the matrix cores accumulate binary16 plus-times in float: by request only, at any size, and with no split-K form
    assert sel(desc(dtype="f16", add="plus", mult="multiplies", m=4096, n=4096)) == b"valu"
    assert ok(desc(dtype="f16", add="plus", mult="multiplies", kernel="mfma")) == 0
    assert sel(desc(dtype="f16", add="plus", mult="multiplies", kernel="mfma")) == b"mfma"
    assert sel(desc(dtype="f16", add="minimum", mult="multiplies")) == b"valu"
    assert sel(desc(dtype="f16", add="logical_or", mult="logical_and")) == b"valu"
    assert sel(desc(dtype="f16", add="plus", mult="maximum")) == b"naive"
    assert cuasr_amd.splitk_workspace_bytes(100, 7, 3, "f16") == 2 * 100 * 7 * 3
    # int8 operands, int32 everything else: A and B at any byte, C and D at four; every integer pair is defined
    d = desc(dtype="i8", add="plus", mult="multiplies")
    assert ok(d) == 0 and sel(d) == b"mfma"
    d.A, d.B = 0x10001, 0x10003
    assert ok(d) == 0
    d.D = 0x10002
    assert ok(d) == 1
    assert sel(desc(dtype="i8")) == b"valu" and ok(desc(dtype="i8", kernel="valu")) == 0   # min-plus: exact in binary16
    assert ok(desc(dtype="i8", add="bit_xor", mult="bit_and")) == 0 and sel(desc(dtype="i8", add="bit_xor", mult="bit_and")) == b"valu"
    assert sel(desc(dtype="i8", add="minimum", mult="multiplies")) == b"valu"      # (int16 lanes)
    assert ok(desc(dtype="i8", add="bit_xor", mult="logical_and")) == 0 and sel(desc(dtype="i8", add="bit_xor", mult="logical_and")) == b"naive"
    assert ok(desc(dtype="i8", add="plus", mult="multiplies", kernel="valu")) == 5
    assert cuasr_amd.splitk_workspace_bytes(100, 7, 3, "i8") == 4 * 100 * 7 * 3
    d = desc()
    d.dtype = 6
    assert ok(d) == 2


def test_kernel_selection(lib):
    sel = lambda d: lib.cuasr_amd_selected_kernel(ctypes.byref(d))
    big = dict(m=4096, n=4096, k=4096)
    assert sel(desc(**big)) == b"valu_direct"      # min-plus f32, aligned, 512 tiles of 256 x 128: direct-to-LDS tile
    assert sel(desc(m=4095, n=4096, k=4096)) == b"valu"   # not vector-sized: staged tile
    assert sel(desc()) == b"valu"                   # 64 x 64: one direct tile would leave the chip idle
    assert sel(desc(m=3072, n=3072, k=64)) == b"valu"     # 288 direct tiles fill 56 % of a round of 512
    assert sel(desc(m=8192, n=8192, k=64)) == b"valu_direct"
    assert sel(desc(add="plus", mult="multiplies", m=2048, n=2048)) == b"mfma"
    assert sel(desc(add="plus", mult="multiplies", m=1024, n=1024)) == b"valu"   # 64 tiles of 128 x 128 leave the chip idle
    assert sel(desc(dtype="f64")) == b"valu"
    assert sel(desc(dtype="f64", m=8192, n=8192, k=64)) == b"valu_direct"   # fp64 direct-to-LDS tile, 128 x 64
    assert sel(desc(dtype="f64", m=2048, n=2048, k=64)) == b"valu_direct"   # 256 of them: one per compute unit is a full round for fp64
    assert sel(desc(m=3072, n=3072, k=4096)) == b"valu_streamk"             # min-plus, half a round of tiles: stream-K ...
    assert sel(desc(m=3072, n=3072, k=4096, mult="maximum")) == b"valu"     # ... but not for the two-instruction min-max
    assert sel(desc(dtype="f64", add="plus", mult="multiplies", m=2048, n=2048)) == b"mfma"   # fp64 matrix cores
    assert sel(desc(dtype="f64", add="plus", mult="multiplies")) == b"valu"
    assert sel(desc(add="plus", mult="bit_or", dtype="i32")) == b"naive"
    assert sel(desc(kernel="mfma")) == b"mfma"
    assert sel(desc(m=5120, n=5120, k=64)) == b"valu_direct+valu"   # 800 direct tiles: one full round + two strips
    assert sel(desc(m=3072, n=3072, k=64)) == b"valu"               # 288 direct tiles fill no round


def test_batched_kernel_selection_looks_at_the_strides(lib):
    """The direct-to-LDS tiles fetch 16-byte vectors, so every product of a batch in the grid has to start at a
    multiple of 16 bytes: strides that do not keep that alignment route the batch to the staged tile."""
    sel = lambda d, batch, *strides: lib.cuasr_amd_selected_kernel_batched(ctypes.byref(d), batch, *strides)
    d = desc(m=512, n=512, k=512)                                   # min-plus f32: 8 direct tiles per product
    whole = 512 * 512
    assert sel(d, 256, whole, whole, whole, whole) == b"valu_direct"
    for odd in range(4):                                            # one stride off by an element is enough
        strides = [whole] * 4
        strides[odd] += 1
        assert sel(d, 256, *strides) == b"valu", odd
        strides[odd] += 3                                           # four floats further: aligned again
        assert sel(d, 256, *strides) == b"valu_direct", odd
    assert sel(d, 256, whole, 0, whole, whole) == b"valu_direct"   # a shared operand (stride 0)
    d = desc(m=512, n=512, k=512, kernel="direct")
    assert sel(d, 256, whole + 1, whole, whole, whole) is None      # asked for by name: refused, not rerouted
    assert lib.cuasr_amd_srgemm_batched(ctypes.byref(d), 256, whole + 1, whole, whole, whole, None) == 1
    d = desc(m=512, n=512, k=512, dtype="f64", add="maximum")
    assert sel(d, 64, whole, whole, whole, whole) == b"valu_direct"
    assert sel(d, 64, whole + 1, whole, whole, whole) == b"valu"    # 8-byte elements: multiples of two
    assert sel(d, 64, whole + 2, whole, whole, whole) == b"valu_direct"
    assert sel(d, 0, whole, whole, whole, whole) is None and sel(d, 4, -1, whole, whole, whole) is None


def test_splitk_host_errors(lib):
    d = desc(m=256, n=256, k=4096, slices=8)
    assert cuasr_amd.splitk_workspace_bytes(256, 256, 8, "f32") == 4 * 256 * 256 * 8
    assert cuasr_amd.splitk_workspace_bytes(100, 7, 3, "f64") == 8 * 100 * 7 * 3
    # null workspace is rejected before anything touches the device
    assert lib.cuasr_amd_srgemm_splitk(ctypes.byref(d), None, None) == 6
    d0 = desc(slices=0)
    assert lib.cuasr_amd_srgemm_splitk(ctypes.byref(d0), ctypes.c_void_p(0x1000), None) == 4
    # the reduction kernel on its own checks its arguments the same way
    assert lib.cuasr_amd_reduce_splitk(ctypes.byref(d), None, None) == 6
    assert lib.cuasr_amd_reduce_splitk(ctypes.byref(d0), ctypes.c_void_p(0x1000), None) == 4
    assert lib.cuasr_amd_reduce_splitk(ctypes.byref(d), ctypes.c_void_p(0x1002), None) == 1
    # the plain entry point refuses split-K descriptors without launching
    assert lib.cuasr_amd_srgemm(ctypes.byref(d), None) == 4


def test_splitk_workspace_alignment_host_side(lib):
    """A workspace aligned to the element but not to 16 bytes: refused for a forced direct-to-LDS tile
    (which stores 16-byte vectors) before anything is launched; 2-byte misalignment refused for every family."""
    d = desc(m=512, n=512, k=4096, slices=8, kernel="direct")
    assert lib.cuasr_amd_srgemm_splitk(ctypes.byref(d), ctypes.c_void_p(0x1004), None) == 1
    assert lib.cuasr_amd_srgemm_splitk_serial(ctypes.byref(d), ctypes.c_void_p(0x1004), None) == 1
    d = desc(m=512, n=512, k=4096, slices=8, dtype="f64", add="maximum", kernel="direct")
    assert lib.cuasr_amd_srgemm_splitk(ctypes.byref(d), ctypes.c_void_p(0x1008), None) == 1
    assert lib.cuasr_amd_srgemm_splitk(ctypes.byref(desc(slices=8)), ctypes.c_void_p(0x1002), None) == 1


def test_static_splitk_host_errors(lib):
    """cuasr_amd_srgemm_splitk_static checks the descriptor and the size of the partial tiles against
    the library's fixed array before it touches the device."""
    call = lambda d: lib.cuasr_amd_srgemm_splitk_static(ctypes.byref(d), None)
    assert cuasr_amd.STATIC_WORKSPACE_BYTES == 16 << 20
    assert lib.cuasr_amd_srgemm_splitk_static(None, None) == 4
    assert call(desc(slices=0)) == 4
    assert call(desc(ptr=0x10002, slices=2)) == 1
    assert call(desc(m=1024, n=1024, k=64, slices=5)) == 10        # 20 MiB of partial tiles: kErrorMemoryAllocation
    assert call(desc(m=2048, n=2048, k=64, slices=1, dtype="f64")) == 10
    assert call(desc(m=46341, n=46341, k=8, slices=2 ** 31 - 1)) == 10   # products past 64 bits are still refused


def test_library_sources_never_allocate():
    """No entry point allocates or frees device memory: nothing in the library's sources names an allocating call."""
    import glob
    import os
    src = os.path.join(os.path.dirname(cuasr_amd.LIB_PATH), "..", "csrc")
    files = glob.glob(os.path.join(src, "*.hip")) + glob.glob(os.path.join(src, "*.h"))
    assert len(files) > 10
    for f in files:
        text = open(f).read()
        for word in ("hipMalloc", "hipFree", "hipHostMalloc", "hipExtMalloc", "hipMemPool", "malloc("):
            assert word not in text, (f, word)


def test_serial_splitk_host_errors(lib):
    # the workspace holds the slices' partial products; none is needed for a single slice (device/srgemm.h:218-234)
    assert cuasr_amd.splitk_serial_workspace_bytes(256, 256, 8, "f32") == 4 * 256 * 256 * 8
    assert cuasr_amd.splitk_serial_workspace_bytes(100, 7, 3, "f64") == 8 * 100 * 7 * 3
    assert cuasr_amd.splitk_serial_workspace_bytes(100, 7, 1, "f64") == 0
    d = desc(m=256, n=256, k=4096, slices=8)
    assert lib.cuasr_amd_srgemm_splitk_serial(ctypes.byref(d), None, None) == 6   # kErrorWorkspaceNull (device/srgemm.h:248-251)
    assert lib.cuasr_amd_srgemm_splitk_serial(ctypes.byref(d), ctypes.c_void_p(0x1002), None) == 1  # misaligned workspace
    d0 = desc(slices=0)
    assert lib.cuasr_amd_srgemm_splitk_serial(ctypes.byref(d0), ctypes.c_void_p(0x1000), None) == 4
    assert lib.cuasr_amd_srgemm_splitk_serial(None, None, None) == 4


def test_fwgemm_host_errors(lib):
    P = ctypes.c_void_p
    call = lambda dtype=0, m=64, n=64, k=64, a=0x1000, lda=64, b=0x1000, ldb=64, d=0x1000, ldc=64, p=0x1000, ldp=64, kern=0: \
        lib.cuasr_amd_fwgemm(dtype, m, n, k, P(a), lda, P(b), ldb, P(d), ldc, P(p), ldp, kern, None)
    assert call(dtype=2) == 2                 # float and double only
    assert call(m=-1) == 4 and call(lda=10) == 4 and call(ldb=63) == 4 and call(ldc=1) == 4 and call(ldp=0) == 4
    assert call(d=0) == 4 and call(p=0) == 4 and call(a=0) == 4
    assert call(a=0x1002) == 1 and call(dtype=1, d=0x1004) == 1 and call(p=0x1001) == 1
    assert call(kern=3) == 5                  # no matrix-core form
    assert call(m=0) == 0 and call(n=0, d=0) == 0 and call(k=0, a=0, b=0) == 0   # nothing to do, nothing launched
    assert cuasr_amd.apsp_workspace_bytes(1000, "f32") == 2 * 4 * 1000 * 1000   # the snapshot and its transpose
    assert cuasr_amd.apsp_workspace_bytes(10, "f64") == 1600 and cuasr_amd.apsp_workspace_bytes(0, "f32") == 0
    sq = lambda n=64, ws=0x1000, it=0, dtype=0: lib.cuasr_amd_apsp_squaring(dtype, n, P(0x1000), max(n, 1), P(0x1000), max(n, 1), P(ws), it, None)
    assert sq(ws=0) == 6 and sq(it=-1) == 4 and sq(dtype=3) == 2 and sq(n=0) == 0
    assert cuasr_amd.apsp_blocked_workspace_bytes(1001, "f32") == 3 * 4 * 128 * (1004 + 128) and cuasr_amd.apsp_blocked_workspace_bytes(0, "f64") == 0
    bl = lambda n=64, ws=0x1000, dtype=0, ld=None: lib.cuasr_amd_apsp_blocked(dtype, n, P(0x1000), ld or max(n, 1), P(0x1000), max(n, 1), P(ws), None)
    assert bl(ws=0) == 6 and bl(dtype=2) == 2 and bl(n=0) == 0 and bl(ld=10) == 4 and bl(ws=0x1004) == 1   # all before any launch
    assert lib.cuasr_amd_apsp_blocked_panels(0, 64, P(0x1000), 64, P(0x1000), 64, P(0x1000), 3, None) == 4   # unknown panel mode
    assert lib.cuasr_amd_apsp_blocked_panels(0, 0, P(0x1000), 1, P(0x1000), 1, P(0x1000), 2, None) == 0


def test_batched_host_errors(lib):
    """Argument checks of the batched call; nothing here launches (a batch of 0 is valid and empty)."""
    d = cuasr_amd.SrgemmDesc()
    d.add_op, d.mult_op, d.dtype = cuasr_amd.OPS["minimum"], cuasr_amd.OPS["plus"], cuasr_amd.DTYPES["f32"]
    d.m = d.n = d.k = 64
    d.split_k_slices = 1
    d.A = d.B = d.C = d.D = 0x1000
    d.lda = d.ldb = d.ldc = d.ldd = 64
    call = lambda batch=0, sa=4096, sb=4096, sc=4096, sd=4096: lib.cuasr_amd_srgemm_batched(
        ctypes.byref(d), batch, sa, sb, sc, sd, None)
    assert call() == 0
    assert call(batch=-1) == 4 and call(sa=-1) == 4 and call(sd=-4096) == 4
    assert call(batch=2, sd=4095) == 4 and call(batch=2, sd=0) == 4      # outputs would overlap
    assert lib.cuasr_amd_srgemm_batched(None, 0, 0, 0, 0, 0, None) == 4
    d.split_k_slices = 2
    assert call() == 4                                                     # as the single call


def test_semiring_constants():
    # include/cuasr/functional.h:28-36, :41-42, :84-85, :127-128, :167-168, :207-208, :247-248
    f32max, f32tiny = np.finfo(np.float32).max, np.finfo(np.float32).tiny
    assert cuasr_amd.op_identity("minimum", "f32") == f32max
    assert cuasr_amd.op_identity("maximum", "f32") == f32tiny          # numeric_limits::min(), not -max
    assert cuasr_amd.op_identity("maximum", "f64") == np.finfo(np.float64).tiny
    assert cuasr_amd.op_annihilator("plus", "f32") == f32max
    assert cuasr_amd.op_identity("maximum", "i32") == np.iinfo(np.int32).min
    assert cuasr_amd.op_identity("plus", "f64") == 0 and cuasr_amd.op_identity("multiplies", "i32") == 1
    assert cuasr_amd.op_identity("logical_and", "i32") == 1 and cuasr_amd.op_annihilator("logical_or", "i32") == 1
    assert cuasr_amd.op_identity("bit_and", "u32") == 0xFFFFFFFF and cuasr_amd.op_identity("bit_xor", "u32") == 0
    assert cuasr_amd.op_identity("minimum", "f32", infinities=True) == np.inf
    assert cuasr_amd.op_identity("maximum", "f64", infinities=True) == -np.inf


def test_inputs_are_reproducible():
    from cuasr_amd import inputs
    a = inputs.uniform(7, 5, 3)
    assert np.array_equal(a, np.asarray(inputs.uniform(7, 5, 3, order="C")))      # same entries in either layout
    assert a.flags["F_CONTIGUOUS"] and a.min() >= 0 and a.max() < 1
    assert inputs.splitmix64(1, 3).tolist() == inputs.splitmix64(1, 5)[:3].tolist()
    g = inputs.graph_distances(1, 64)
    assert np.all(np.diag(g) == 0) and np.isinf(g).mean() > 0.8
    w = inputs.words32(3, 64, 64)
    assert w.dtype == np.uint32 and 0.4 < np.unpackbits(np.ascontiguousarray(w).view(np.uint8)).mean() < 0.6


def test_user_functor_without_hipcc_is_a_readable_compile_error(tmp_path):
    """A functor that is none of the library's operators needs its kernel built from the functor: with a
    host-only compiler device::Srgemm::run must stop the build with a message that says what to do."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "user.cpp"
    src.write_text("""
#include "cuasr/gemm/device/srgemm.h"
template <typename T, int N = 1> struct my_op {
  static constexpr T Identity = 0, Annihilator = 0;
  T operator()(T l, T const &r) const { return l + 2 * r; }
};
int main() {
  using L = cuasr::layout::ColumnMajor;
  cuasr::gemm::device::Srgemm<my_op<float>, cuasr::plus<float>, float, L, float, L, float, L, float> op;
  return (int)op.run();
}
""")
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I", "/opt/rocm/include",
           "-I", os.path.join(root, "include"), str(src)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode != 0
    assert "compile this translation unit with hipcc" in r.stderr
    # the same program with library functors compiles with the host compiler alone
    src.write_text(src.read_text().replace("my_op<float>", "cuasr::minimum<float>"))
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]


def test_reference_call_sites_compile():
    """A program that spells its operators the way the reference's examples do (cutlass:: names, a user functor
    with Array overloads, split-K with an owning workspace buffer) compiles against this library's headers --
    hipcc cross-compiles it here; tests/test_gpu_cpp_api.py runs it on the GPU."""
    import build_cpp
    assert os.path.exists(build_cpp.build("test_reference_call_sites"))
