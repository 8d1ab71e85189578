"""First GPU parity checks: every kernel family against the CPU oracle,
bit-exact, through the C ABI."""
import numpy as np
import pytest

from helpers import assert_same_bits, order_of, to_device, to_host

pytestmark = pytest.mark.gpu


def run(oracle, add, mult, dtype, m, n, k, la, lb, lc, kernel, beta_one, seed=1, inf=True, splitk=0):
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    npd = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "u32": np.uint32}[dtype]
    if dtype in ("f32", "f64"):
        A = inputs.integers(seed, m, k, -8, 8, npd, order_of(la))
        B = inputs.integers(seed + 1, k, n, -8, 8, npd, order_of(lb))
        C = inputs.integers(seed + 2, m, n, -8, 8, npd, order_of(lc))
    elif {add, mult} & {"plus", "multiplies", "minimum", "maximum"}:
        # arithmetic on integers: small values, so nothing overflows (signed overflow is undefined on the CPU side)
        A = inputs.integers(seed, m, k, 0, 8, npd, order_of(la))
        B = inputs.integers(seed + 1, k, n, 0, 8, npd, order_of(lb))
        C = inputs.integers(seed + 2, m, n, 0, 8, npd, order_of(lc))
    else:
        A = inputs.words32(seed, m, k, order_of(la)).astype(npd)
        B = inputs.words32(seed + 1, k, n, order_of(lb)).astype(npd)
        C = inputs.words32(seed + 2, m, n, order_of(lc)).astype(npd)
    ident = cuasr_amd.op_identity(add, dtype, inf)
    one = cuasr_amd.op_identity(mult, dtype, inf)
    zero = cuasr_amd.op_annihilator(mult, dtype, inf)
    if add == "maximum" and mult == "plus":
        zero = ident  # the max-semiring zero, not plus::Annihilator
    alpha, beta = one, (one if beta_one else zero)
    want = oracle.srgemm(add, mult, A, B, C, alpha, beta, ident)
    dA, dB, dC = to_device(A), to_device(B), to_device(C)
    dD = to_device(np.zeros_like(C))
    if splitk:
        ws = torch.empty(cuasr_amd.splitk_workspace_bytes(m, n, splitk, dtype) // 4 + 4, dtype=torch.int32, device="cuda")
        cuasr_amd.srgemm_splitk(add, mult, dA, dB, dC, dD, splitk, ws, alpha, beta, ident, one, dtype=dtype, kernel=kernel)
    else:
        cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, alpha, beta, ident, one, dtype=dtype, kernel=kernel)
    torch.cuda.synchronize()
    assert_same_bits(to_host(dD, dtype), want, f"{add}-{mult} {dtype} {m}x{n}x{k} {la}{lb}{lc} {kernel}")


@pytest.mark.parametrize("kernel", ["naive", "valu"])
@pytest.mark.parametrize("shape", [(1, 1, 1), (17, 27, 17), (128, 128, 64), (256, 384, 100), (509, 510, 23)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_minplus_f32(oracle, lib, kernel, shape, layouts):
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for beta_one in (False, True):
        run(oracle, "minimum", "plus", "f32", *shape, la, lb, lc, kernel, beta_one)


@pytest.mark.parametrize("kernel", ["naive", "valu"])
@pytest.mark.parametrize("sr", [("maximum", "plus", "f64"), ("maximum", "minimum", "f64"), ("plus", "multiplies", "f32"),
                                ("bit_xor", "bit_and", "u32"), ("logical_or", "logical_and", "i32")])
def test_other_semirings(oracle, lib, kernel, sr):
    for shape in [(128, 64, 32), (130, 70, 37), (256, 256, 256)]:
        for layouts in ("ccc", "rcr"):
            la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
            run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, kernel, True)


@pytest.mark.parametrize("sr", [("minimum", "plus", "f32"), ("maximum", "plus", "f64"), ("maximum", "minimum", "f64"),
                                ("plus", "multiplies", "f32"), ("bit_xor", "bit_and", "u32"), ("minimum", "plus", "i32")])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_valu_full_size_tile(oracle, lib, sr, layouts):
    """The staged family uses its quarter-size tile unless the full-size one fills its rounds; these grids are
    whole rounds of 1024 workgroups (>= 95 % filled) for the full-size tile, ragged edges included."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for shape in [(4096, 4096, 40), (4090, 4000, 19)]:
        run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, "valu", True)


def test_valu_splitk_tile_sizes(oracle, lib):
    """Split-K through both tile sizes of the staged family: 4 tiles x 8 slices (quarter-size tile)
    and 4 tiles x 256 slices (full-size tile)."""
    for slices in (8, 256):
        run(oracle, "minimum", "plus", "f32", 256, 256, 4096, "row", "col", "row", "valu", True, splitk=slices)
        run(oracle, "maximum", "plus", "f64", 256, 256, 2048, "col", "col", "col", "valu", False, splitk=slices)


@pytest.mark.parametrize("sr", [("minimum", "plus", "f32"), ("maximum", "plus", "f64"), ("bit_xor", "bit_and", "u32"),
                                ("plus", "multiplies", "f32")])
def test_splitk_large_output(oracle, lib, sr):
    """Outputs of a million elements and more take the reduction kernel's 16-byte path
    (smaller ones its one-element-per-thread path); small integers keep plus-times exact."""
    for layouts in ("rcr", "ccc"):
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        run(oracle, sr[0], sr[1], sr[2], 1024, 1280, 96, la, lb, lc, "auto", True, splitk=3)
        run(oracle, sr[0], sr[1], sr[2], 1024, 1280, 96, la, lb, lc, "valu", False, splitk=5)


@pytest.mark.parametrize("kernel", ["naive", "valu"])
@pytest.mark.parametrize("slices", [1, 3, 8])
def test_splitk_minplus(oracle, lib, kernel, slices):
    run(oracle, "minimum", "plus", "f32", 128, 128, 1000, "row", "col", "row", kernel, False, splitk=slices)
    run(oracle, "minimum", "plus", "f32", 100, 60, 333, "col", "col", "col", kernel, True, splitk=slices)


@pytest.mark.parametrize("add", ["minimum", "maximum"])
@pytest.mark.parametrize("shape", [(128, 128, 16), (128, 128, 64), (256, 384, 100), (64, 4, 8), (4, 4, 4),
                                   (516, 260, 52), (1024, 1024, 1024)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_tropical_mfma(oracle, lib, add, shape, layouts):
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for beta_one in (False, True):
        run(oracle, add, "plus", "f32", *shape, la, lb, lc, "mfma", beta_one)


@pytest.mark.parametrize("slices", [1, 3, 8])
def test_splitk_mfma(oracle, lib, slices):
    run(oracle, "minimum", "plus", "f32", 128, 128, 1000, "row", "col", "row", "mfma", False, splitk=slices)
    run(oracle, "minimum", "plus", "f32", 100, 60, 332, "col", "col", "col", "mfma", True, splitk=slices)


def test_minplus_uniform_1024(oracle, lib):
    """min-plus f32 1024^3, all column-major, uniform [0,1), identity +inf."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    n = 1024
    A = inputs.uniform(11, n, n)
    B = inputs.uniform(12, n, n)
    C = np.full((n, n), np.inf, dtype=np.float32, order="F")
    want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, np.inf, np.inf)
    for kernel in ("auto", "valu", "naive"):
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm("minimum", "plus", to_device(A), to_device(B), to_device(C), dD, 0.0, np.inf, np.inf, 0.0, kernel=kernel)
        torch.cuda.synchronize()
        assert_same_bits(to_host(dD, "f32"), want, kernel)


@pytest.mark.parametrize("sr", [("minimum", "plus", "f32"), ("maximum", "plus", "f32"), ("plus", "multiplies", "f32"),
                                ("maximum", "minimum", "f32"), ("bit_xor", "bit_and", "u32"), ("minimum", "plus", "i32"),
                                ("maximum", "plus", "f64"), ("maximum", "minimum", "f64"), ("plus", "multiplies", "f64")])
@pytest.mark.parametrize("shape", [(128, 128, 16), (128, 128, 64), (256, 384, 100), (64, 4, 8), (4, 4, 4),
                                   (516, 260, 52), (132, 388, 1028), (1024, 1024, 1024)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr", "rcc", "crr", "ccr", "rrc"])
def test_direct_tile(oracle, lib, sr, shape, layouts):
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    if shape[0] >= 1024 and layouts not in ("ccc", "rcr", "crr"):
        pytest.skip("large shape: three layout combinations are enough")
    for beta_one in (False, True):
        if not beta_one and sr[2] == "i32" and sr[1] == "plus":
            continue  # plus::Annihilator = INT_MAX: mult(beta, c) overflows on the CPU side (undefined)
        run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, "direct", beta_one)


@pytest.mark.parametrize("sr", [("bit_xor", "bit_and", "u32"), ("bit_or", "bit_and", "u32"), ("bit_xor", "bit_and", "i32")])
@pytest.mark.parametrize("shape", [(256, 128, 16), (256, 128, 32), (260, 132, 48), (516, 388, 160), (1024, 1024, 1024), (12, 8, 64)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr", "rcc", "crr", "ccr", "rrc"])
def test_direct_tile_on_words(oracle, lib, sr, shape, layouts):
    """xor-and / or-and on 32-bit words with k a multiple of 16 on the direct-to-LDS tile: one, two, three and
    many k-tiles (every depth of its three-stage prologue), ragged edges in m and n, an output smaller than a
    tile, every layout combination."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    if shape[0] >= 1024 and layouts not in ("ccc", "rcr", "crr", "rrr"):
        pytest.skip("large shape: four layout combinations are enough")
    for beta_one in (False, True):
        run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, "direct", beta_one)


def test_direct_tile_on_words_splitk(oracle, lib):
    run(oracle, "bit_xor", "bit_and", "u32", 260, 132, 512, "col", "col", "col", "direct", True, splitk=4)
    run(oracle, "bit_or", "bit_and", "u32", 256, 256, 1024, "row", "row", "row", "direct", False, splitk=8)


@pytest.mark.parametrize("slices", [1, 3, 8])
def test_splitk_direct(oracle, lib, slices):
    run(oracle, "minimum", "plus", "f32", 128, 128, 1000, "row", "col", "row", "direct", False, splitk=slices)
    run(oracle, "minimum", "plus", "f32", 100, 60, 332, "col", "col", "col", "direct", True, splitk=slices)
    run(oracle, "bit_xor", "bit_and", "u32", 260, 132, 520, "col", "row", "row", "direct", True, splitk=slices)
    run(oracle, "maximum", "plus", "f64", 260, 132, 520, "col", "row", "row", "direct", True, splitk=slices)
    run(oracle, "maximum", "minimum", "f64", 128, 64, 1000, "row", "col", "row", "direct", False, splitk=slices)


@pytest.mark.parametrize("shape", [(128, 128, 16), (256, 384, 100), (64, 4, 8), (516, 260, 52), (1024, 1024, 1024)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_plus_times_mfma_small_integers(oracle, lib, shape, layouts):
    """Matrix-core plus-times on small integers: every partial sum is exact in fp32, so any summation
    order gives the host reference's bits (the reference's own testbed relies on the same fact)."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for beta_one in (False, True):
        run(oracle, "plus", "multiplies", "f32", *shape, la, lb, lc, "mfma", beta_one)


@pytest.mark.parametrize("shape", [(1001, 997, 333), (130, 66, 6), (257, 129, 17), (1, 1, 1), (3, 5, 2), (2501, 2303, 70), (63, 1, 5)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr", "rcc", "crr", "ccr", "rrc"])
def test_plus_times_mfma_any_extent(oracle, lib, shape, layouts):
    """Extents, leading dimensions and k that are not multiples of the 16-byte vector: the matrix-core kernels'
    element-aligned forms (vectors that would cross the end of a row or of the k range are read element by
    element), float and double.  Small integers, so the host reference's bits are the answer."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for dtype in ("f32", "f64"):
        for beta_one in (False, True):
            run(oracle, "plus", "multiplies", dtype, *shape, la, lb, lc, "mfma", beta_one)
        if shape[2] > 64:
            run(oracle, "plus", "multiplies", dtype, *shape, la, lb, lc, "mfma", True, splitk=3)


@pytest.mark.parametrize("shape", [(3584, 4096, 16), (3588, 4092, 48), (3588, 4092, 160), (3584, 4096, 32)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_plus_times_mfma_hand_scheduled(oracle, lib, shape, layouts):
    """Outputs that fill a round of 128 x 256 tiles with k a multiple of 16 take the hand-scheduled
    matrix-core loop (one, two, three and ten k-tiles: every depth of its three-stage prologue; ragged
    edges in m and n); small integers, so the host reference's bits are the answer."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    run(oracle, "plus", "multiplies", "f32", *shape, la, lb, lc, "mfma", shape[2] == 48)


@pytest.mark.parametrize("shape", [(2048, 2048, 16), (2052, 2044, 48), (1156, 1284, 160), (2048, 2048, 32)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_plus_times_mfma_hand_scheduled_narrow_tile(oracle, lib, shape, layouts):
    """Outputs whose 128 x 256 tiles would leave most of a round empty take the 128 x 128 form of the
    hand-scheduled loop; same cases as for the wide one."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    run(oracle, "plus", "multiplies", "f32", *shape, la, lb, lc, "mfma", shape[2] == 48)


def test_plus_times_mfma_hand_scheduled_splitk(oracle, lib):
    run(oracle, "plus", "multiplies", "f32", 1024, 1024, 512, "row", "col", "row", "mfma", True, splitk=16)
    run(oracle, "plus", "multiplies", "f32", 1024, 1024, 1024, "col", "row", "col", "mfma", False, splitk=16)


def test_plus_times_mfma_splitk(oracle, lib):
    run(oracle, "plus", "multiplies", "f32", 128, 128, 1000, "row", "col", "row", "mfma", True, splitk=8)
    run(oracle, "plus", "multiplies", "f32", 100, 60, 332, "col", "col", "col", "mfma", True, splitk=3)


@pytest.mark.parametrize("shape", [(128, 128, 16), (256, 384, 100), (64, 4, 8), (516, 260, 50), (130, 66, 6), (1024, 1024, 1024)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_plus_times_mfma_f64_small_integers(oracle, lib, shape, layouts):
    """fp64 matrix-core plus-times on small integers: every partial sum is exact, so any summation
    order gives the host reference's bits."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for beta_one in (False, True):
        run(oracle, "plus", "multiplies", "f64", *shape, la, lb, lc, "mfma", beta_one)


@pytest.mark.parametrize("shape", [(3584, 2048, 16), (3586, 2046, 48), (3586, 2046, 160), (3584, 2048, 32)])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_plus_times_mfma_f64_hand_scheduled(oracle, lib, shape, layouts):
    """Outputs that fill a round of 128 x 128 tiles with k a multiple of 16 take the hand-scheduled fp64
    matrix-core loop (one, two, three and ten k-tiles; ragged edges in m and n); small integers, so the
    host reference's bits are the answer."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    run(oracle, "plus", "multiplies", "f64", *shape, la, lb, lc, "mfma", shape[2] == 48)


def test_plus_times_mfma_f64_hand_scheduled_splitk(oracle, lib):
    run(oracle, "plus", "multiplies", "f64", 1024, 1024, 512, "row", "col", "row", "mfma", True, splitk=8)
    run(oracle, "plus", "multiplies", "f64", 1024, 1024, 1024, "col", "row", "col", "mfma", False, splitk=8)


def test_plus_times_mfma_f64_splitk(oracle, lib):
    run(oracle, "plus", "multiplies", "f64", 128, 128, 1000, "row", "col", "row", "mfma", True, splitk=8)
    run(oracle, "plus", "multiplies", "f64", 100, 60, 332, "col", "col", "col", "mfma", True, splitk=3)


def test_plus_times_f64_tolerance(oracle, lib):
    """fp64 plus-times on N(0,1) data, default kernel (matrix cores): within 1e-12 relative of the host
    reference -- per element against sum_k |a||b| and in the Frobenius norm; the vector-ALU tile bit-exact."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    m, n, k = 512, 384, 2048
    A = inputs.normal(701, m, k).astype(np.float64) + 1e-9 * inputs.normal(703, m, k).astype(np.float64)
    B = inputs.normal(702, k, n).astype(np.float64) + 1e-9 * inputs.normal(704, k, n).astype(np.float64)
    A, B = np.asfortranarray(A), np.asfortranarray(B)
    C = np.zeros((m, n), dtype=np.float64, order="F")
    want = oracle.srgemm("plus", "multiplies", A, B, C, 1.0, 0.0, 0.0)
    for kernel, exact in (("auto", False), ("valu", True)):
        dD = to_device(np.zeros_like(C))
        cuasr_amd.srgemm("plus", "multiplies", to_device(A), to_device(B), to_device(C), dD, 1.0, 0.0, 0.0, 1.0,
                         dtype="f64", kernel=kernel)
        torch.cuda.synchronize()
        got = to_host(dD, "f64")
        if exact:
            assert_same_bits(got, want, "vector-ALU fp64 plus-times")
        else:
            diff = np.abs(got - want)
            assert np.all(diff <= 1e-12 * (np.abs(A) @ np.abs(B)))          # tolerance 1e-12 relative
            assert np.linalg.norm(diff) <= 1e-12 * np.linalg.norm(want)


@pytest.mark.parametrize("sr", [("minimum", "plus", "f32"), ("maximum", "plus", "f64"), ("plus", "multiplies", "f32"),
                                ("bit_xor", "bit_and", "u32")])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "rcr"])
def test_unaligned_views(oracle, lib, sr, layouts):
    """Operands that are interior windows of larger buffers: base pointers aligned to the element only,
    leading dimensions larger than the extents and odd, extents not multiples of the vector width.
    Every kernel family AUTO may pick and the staged family itself must reproduce the oracle."""
    import torch
    import cuasr_amd
    from cuasr_amd import inputs
    add, mult, dtype = sr
    npd = {"f32": np.float32, "f64": np.float64, "u32": np.uint32}[dtype]
    for (m, n, k) in [(131, 67, 45), (515, 262, 131), (1027, 1030, 77)]:
        def window(seed, rows, cols, layout):
            # a (rows x cols) window at offset (3, 1) of a buffer with 5 spare rows and 7 spare columns
            R, Cc = rows + 5, cols + 7
            if dtype == "u32":
                full = inputs.words32(seed, R, Cc, "C")
            else:
                full = inputs.integers(seed, R, Cc, -8, 8, npd, "C")
            host = full[3:3 + rows, 1:1 + cols]
            if layout == "row":
                dev = torch.from_numpy(full.view(np.int32) if dtype == "u32" else full).cuda()[3:3 + rows, 1:1 + cols]
            else:  # column-major window: transpose view of a row-major buffer holding the transpose
                fullT = np.ascontiguousarray(full.T)
                dev = torch.from_numpy(fullT.view(np.int32) if dtype == "u32" else fullT).cuda()[1:1 + cols, 3:3 + rows].t()
            return host, dev
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        A, dA = window(31, m, k, la)
        B, dB = window(32, k, n, lb)
        C, dC = window(33, m, n, lc)
        _, dD0 = window(34, m, n, lc)
        ident = cuasr_amd.op_identity(add, dtype, True)
        one = cuasr_amd.op_identity(mult, dtype, True)
        order = "F" if lc == "col" else "C"
        want = oracle.srgemm(add, mult, np.asarray(A, order=("F" if la == "col" else "C")), np.asarray(B, order=("F" if lb == "col" else "C")),
                             np.asarray(C, order=order), one, one, ident)
        # (plus-times on the matrix cores has an element-aligned form for such operands)
        for kernel in ("auto", "valu") + (("mfma",) if (add, mult, dtype) == ("plus", "multiplies", "f32") else ()):
            dD = dD0.clone() if False else dD0  # the window of D is written in place
            cuasr_amd.srgemm(add, mult, dA, dB, dC, dD, one, one, ident, one, dtype=dtype, kernel=kernel)
            torch.cuda.synchronize()
            assert_same_bits(np.asarray(to_host(dD, dtype), order=order), want, f"{sr} {layouts} {m}x{n}x{k} {kernel}")


@pytest.mark.parametrize("sr", [("minimum", "plus", "f32"), ("maximum", "plus", "f64"), ("bit_xor", "bit_and", "u32"),
                                ("logical_or", "logical_and", "f32"), ("minimum", "multiplies", "f32"),
                                ("maximum", "minimum", "f64"), ("minimum", "plus", "i32"), ("plus", "multiplies", "f32")])
@pytest.mark.parametrize("shape", [(64, 64, 256), (100, 60, 1000), (256, 256, 4099), (512, 512, 512), (1024, 1024, 1024),
                                   (1000, 1100, 300), (61, 67, 1027)])
def test_valu_small_launches_share_k_inside_the_workgroup(oracle, lib, sr, shape):
    """Launches of at most 512 quarter-size tiles with a long enough k range run two or four groups of 256 threads
    per workgroup, each on a part of the k range (every add but a floating-point sum); results stay the reference's."""
    for layouts in ("ccc", "rcr", "crr", "rrc"):
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        if shape[0] >= 1000 and layouts in ("crr", "rrc"):
            continue
        for beta_one in (False, True):
            if not beta_one and sr[2] == "i32" and sr[1] == "plus":
                continue  # plus::Annihilator = INT_MAX: mult(beta, c) overflows on the CPU side (undefined)
            run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, "valu", beta_one)
    run(oracle, sr[0], sr[1], sr[2], *shape, "row", "col", "row", "valu", True, splitk=3)


@pytest.mark.parametrize("sr", [("minimum", "plus", "f32"), ("maximum", "plus", "f64"), ("bit_xor", "bit_and", "u32"),
                                ("logical_or", "logical_and", "f32"), ("minimum", "multiplies", "f64"),
                                ("maximum", "minimum", "f32"), ("plus", "multiplies", "f32")])
@pytest.mark.parametrize("shape", [(2048, 2048, 260), (1792, 1920, 300), (2048, 1024, 300), (2040, 2047, 517)])
def test_valu_full_size_tile_two_groups(oracle, lib, sr, shape):
    """192 .. 256 full-size tiles (one workgroup per compute unit): two groups of 256 threads per workgroup
    share the k range (every add but a floating-point sum)."""
    for layouts in ("ccc", "rcr"):
        la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
        run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, "valu", True)
    run(oracle, sr[0], sr[1], sr[2], *shape, "col", "row", "row", "valu", False)


@pytest.mark.parametrize("case", [("minimum", "plus", "f32", 5120, 5120, 24, "ccc"), ("minimum", "plus", "f32", 5120, 4736, 20, "rcr"),
                                  ("bit_xor", "bit_and", "u32", 4608, 5248, 16, "crr"), ("maximum", "plus", "f64", 4480, 3264, 12, "ccc"),
                                  ("plus", "multiplies", "f32", 5124, 5000, 8, "ccr")])
def test_large_output_in_two_regions(oracle, lib, case):
    """Outputs whose direct-to-LDS tiles do not fill whole rounds run a top-left block on that tile and the two
    remaining strips on the staged tiles: three launches, disjoint parts of D."""
    add, mult, dtype, m, n, k, layouts = case
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for beta_one in (True, False):
        run(oracle, add, mult, dtype, m, n, k, la, lb, lc, "auto", beta_one)


STREAMK_SEMIRINGS = [("minimum", "plus", "f32"), ("maximum", "plus", "f32"), ("maximum", "minimum", "f32"),
                     ("minimum", "maximum", "f32"), ("bit_xor", "bit_and", "u32"), ("bit_or", "bit_and", "i32")]


@pytest.mark.parametrize("sr", STREAMK_SEMIRINGS)
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc", "crr", "ccr", "rrc"])
def test_streamk_direct_tile(oracle, lib, sr, layouts):
    """The direct tile with the k-tiles of all output tiles shared out over the workgroups: ranges of k of one
    tile meet in D (plain fold for a workgroup that has a tile to itself, atomic folds otherwise).  Shapes of
    one tile, of a few tiles with far more workgroups than tiles (every tile split many ways), ragged edges and
    a ragged last k-tile; beta = zero (D starts from the identity) and beta = one (from the source)."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for shape in [(128, 128, 64), (256, 384, 100), (516, 260, 52), (132, 388, 1028), (768, 640, 4096)]:
        for beta_one in (False, True):
            run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, "streamk", beta_one)


@pytest.mark.parametrize("sr", [("minimum", "plus", "f32"), ("bit_xor", "bit_and", "u32")])
@pytest.mark.parametrize("layouts", ["ccc", "rrr", "crc"])
def test_streamk_more_tiles_than_workgroups(oracle, lib, sr, layouts):
    """561 and 1100 tiles for 512 workgroups: whole tiles first (one and two per workgroup), the rest shared."""
    la, lb, lc = [{"c": "col", "r": "row"}[x] for x in layouts]
    for shape in [(4352, 4224, 48), (5632, 6400, 36)]:
        run(oracle, sr[0], sr[1], sr[2], *shape, la, lb, lc, "streamk", True)


def test_streamk_is_what_auto_picks_for_half_filled_rounds(oracle, lib):
    """3072 x 3072 is 288 tiles for 512 places; AUTO takes the stream-K form there, and not for 4096^2 (512 tiles), a
    pair of k-contiguous operands, a short k, or an alpha that is not the multiplicative identity."""
    import ctypes
    import cuasr_amd
    from cuasr_amd import COLUMN_MAJOR, ROW_MAJOR, MatRef

    def chosen(m, n, k, la=COLUMN_MAJOR, lb=COLUMN_MAJOR, alpha=0.0, add="minimum", mult="plus"):
        A = MatRef(0x10000, m if la == COLUMN_MAJOR else k, la, m, k)
        B = MatRef(0x10000, k if lb == COLUMN_MAJOR else n, lb, k, n)
        C = MatRef(0x10000, m, COLUMN_MAJOR, m, n)
        d = cuasr_amd.make_desc(add, mult, "f32", A, B, C, C, alpha, 0.0, float("inf"), 0.0)
        return lib.cuasr_amd_selected_kernel(ctypes.byref(d))
    assert chosen(3072, 3072, 3072) == b"valu_streamk"
    assert chosen(5120, 5120, 5120) == b"valu_streamk"
    assert chosen(4096, 4096, 4096) == b"valu_direct"
    assert chosen(3072, 3072, 64) != b"valu_streamk"
    assert chosen(3072, 3072, 3072, alpha=1.0) != b"valu_streamk"
    assert chosen(3072, 3072, 3072, la=ROW_MAJOR, lb=COLUMN_MAJOR) != b"valu_streamk"   # both operands k-contiguous: no such loop
    assert chosen(3072, 3072, 3072, la=COLUMN_MAJOR, lb=ROW_MAJOR) == b"valu_streamk"
    assert chosen(3072, 3072, 3072, add="plus", mult="multiplies") != b"valu_streamk"
    run(oracle, "minimum", "plus", "f32", 3072, 3072, 1024, "col", "col", "col", "auto", True)
