"""Pins the CPU oracle (oracle/host_srgemm.c) without running any reference code:
the reference's own known-answer vector, a literal pure-Python triple loop on
ragged shapes / all layouts / every operator pair, and closed forms the
mathematics fixes (GEMM, GF(2) bit planes, boolean reachability, Floyd-Warshall
shortest paths, widest paths)."""
import itertools
import json
import os

import numpy as np
import pytest

from cuasr_amd import inputs
from helpers import assert_same_bits

HERE = os.path.dirname(os.path.abspath(__file__))

PY_OPS = {
    "plus": lambda l, r: l + r,
    "multiplies": lambda l, r: l * r,
    "minimum": lambda l, r: r if r < l else l,
    "maximum": lambda l, r: r if l < r else l,
    "logical_and": lambda l, r: type(l)(bool(l) and bool(r)),
    "logical_or": lambda l, r: type(l)(bool(l) or bool(r)),
    "bit_and": lambda l, r: l & r,
    "bit_or": lambda l, r: l | r,
    "bit_xor": lambda l, r: l ^ r,
}


def literal_srgemm(add, mult, A, B, C, alpha, beta, ident):
    """The reference host loop, literally (host_srgemm.h:75-109), in Python scalars
    of the matrix dtype: accum = add(mult(a, b), accum), then
    D = add(mult(alpha, accum), mult(beta, c))."""
    f_add, f_mul = PY_OPS[add], PY_OPS[mult]
    t = A.dtype.type
    m, k = A.shape
    n = B.shape[1]
    D = np.empty((m, n), dtype=A.dtype)
    with np.errstate(over="ignore"):
        for i in range(m):
            for j in range(n):
                acc = t(ident)
                for kk in range(k):
                    acc = t(f_add(t(f_mul(A[i, kk], B[kk, j])), acc))
                D[i, j] = t(f_add(t(f_mul(t(alpha), acc)), t(f_mul(t(beta), C[i, j]))))
    return D


def bits(x):
    return np.ascontiguousarray(x).tobytes()


def test_reference_known_answer_vector(oracle):
    g = json.load(open(os.path.join(HERE, "golden", "regress_minplus_4x4x2.json")))
    f = lambda key, r, c: np.array(g[key], dtype=np.float32).reshape(c, r).T
    A, B, C = f("a_colmajor", 4, 2), f("b_colmajor", 2, 4), f("c_colmajor", 4, 4)
    want = f("expected_colmajor", 4, 4)
    for naive in (False, True):
        for order in ("F", "C"):
            got = oracle.srgemm("minimum", "plus", np.asarray(A, order=order), np.asarray(B, order=order),
                                np.asarray(C, order=order), 0.0, 0.0, np.finfo(np.float32).max, naive=naive)
            # the reference compares with EXPECT_FLOAT_EQ (4 ulp); the literals round-trip exactly
            assert np.array_equal(got, want)
    # only linear index 11 (column-major) differs from C, as in the reference test
    diff = np.flatnonzero(want.T.ravel() != C.T.ravel())
    assert diff.tolist() == [11]


FLOAT_PAIRS = [("plus", "multiplies"), ("minimum", "plus"), ("maximum", "plus"), ("minimum", "multiplies"),
               ("maximum", "multiplies"), ("minimum", "maximum"), ("maximum", "minimum"), ("logical_or", "logical_and")]
INT_PAIRS = FLOAT_PAIRS + [("bit_xor", "bit_and"), ("bit_xor", "logical_and"), ("bit_or", "bit_and")]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int32, np.uint32, np.float16])
@pytest.mark.parametrize("shape", [(1, 1, 1), (7, 6, 5), (17, 27, 17), (33, 34, 3)])
def test_against_literal_loop(oracle, dtype, shape):
    m, n, k = shape
    pairs = FLOAT_PAIRS if np.dtype(dtype).kind == "f" else INT_PAIRS
    lo = 0 if np.dtype(dtype).kind == "u" else -8
    for (add, mult), (la, lb, lc) in zip(pairs, itertools.cycle(itertools.product("FC", repeat=3))):
        A = inputs.integers(5, m, k, lo, 8, dtype, la)
        B = inputs.integers(6, k, n, lo, 8, dtype, lb)
        C = inputs.integers(7, m, n, lo, 8, dtype, lc)
        for alpha, beta, ident in [(1, 0, 0), (1, 1, 3), (2, 1, 5)]:
            want = literal_srgemm(add, mult, A, B, C, alpha, beta, ident)
            for naive in (False, True):
                got = oracle.srgemm(add, mult, A, B, C, alpha, beta, ident, naive=naive)
                assert bits(got) == bits(np.asarray(want, order=lc)), (add, mult, la, lb, lc, naive)


def test_binary16_conversions_match_numpy(oracle):
    """The oracle holds binary16 as bit patterns and converts by hand (its compiler has no half type):
    every one of the 65536 patterns widens as numpy's float16 does, and narrowing rounds to nearest even
    on random binary32 values, on every midpoint between neighbouring binary16 values and on the values
    next to each midpoint (where a wrong tie rule or a dropped sticky bit shows)."""
    import ctypes
    lib = oracle.lib()
    lib.oracle_half_to_float.restype, lib.oracle_half_to_float.argtypes = ctypes.c_float, [ctypes.c_uint16]
    lib.oracle_float_to_half.restype, lib.oracle_float_to_half.argtypes = ctypes.c_uint16, [ctypes.c_float]
    every = np.arange(65536, dtype=np.uint16)
    want = every.view(np.float16).astype(np.float32)
    got = np.array([lib.oracle_half_to_float(int(h)) for h in every], dtype=np.float32)
    finite = ~np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[finite], want.view(np.uint32)[finite]) and np.isnan(got[~finite]).all()
    halves = np.arange(0, 0x7c01, dtype=np.uint16).view(np.float16).astype(np.float64)   # 0 .. 65504, then inf
    halves[-1] = 65536.0                                                                  # the value binary16 would hold next
    mids = ((halves[:-1] + halves[1:]) / 2).astype(np.float32)                            # exact in binary32
    near = np.concatenate([mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9))])
    rnd = inputs.splitmix64(11, 60000).astype(np.uint32).view(np.float32)
    f = np.concatenate([near, -near, rnd, np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.99, 65520.0, 1e30], np.float32)])
    f = f[~np.isnan(f)]
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([lib.oracle_float_to_half(float(x)) for x in f], dtype=np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("pair", FLOAT_PAIRS)
def test_binary16_every_operator_rounds_once(oracle, pair):
    """Values whose sums and products do not fit binary16: the oracle against the literal loop on numpy
    float16 scalars (numpy rounds each float16 operation once, to nearest even), both oracle loops."""
    add, mult = pair
    m, n, k = 9, 10, 37
    lo, hi = (-2.0, 2.0) if mult == "multiplies" else (-300.0, 300.0)
    A = inputs.uniform(21, m, k, lo, hi, np.float16, "F")
    B = inputs.uniform(22, k, n, lo, hi, np.float16, "C")
    C = inputs.uniform(23, m, n, lo, hi, np.float16, "F")
    A[0, :5] = np.float16(6e-5) * np.arange(5, dtype=np.float16)      # subnormal operands and results
    B[:5, 0] = np.float16(3e-4)
    for alpha, beta, ident in [(1.0, 0.0, 0.0), (0.7, 1.3, np.inf), (1.0, 1.0, -np.inf), (3.0, 0.25, 65504.0)]:
        want = literal_srgemm(add, mult, A, B, C, np.float16(alpha), np.float16(beta), np.float16(ident))
        for naive in (False, True):
            got = oracle.srgemm(add, mult, A, B, C, np.float16(alpha), np.float16(beta), np.float16(ident), naive=naive)
            nan = np.isnan(want)      # (inf - inf in max-plus with a -inf identity: any NaN will do)
            assert np.array_equal(np.isnan(got), nan)
            assert bits(np.where(nan, 0, got)) == bits(np.where(nan, 0, np.asarray(want, order="F"))), (add, mult, alpha, beta, ident, naive)


def test_binary16_shortest_paths_on_small_integers(oracle):
    """Integer weights whose path sums stay below 2048 are exact in binary16: repeated min-plus squaring
    in half precision gives Floyd-Warshall's distances."""
    n = 60
    rng = np.random.default_rng(5)
    W = np.where(rng.random((n, n)) < 0.2, rng.integers(1, 9, (n, n)), np.inf)
    np.fill_diagonal(W, 0)
    want = floyd_warshall(W.copy())
    assert want[np.isfinite(want)].max() < 2048
    D = np.asfortranarray(W.astype(np.float16))
    inf = np.float16(np.inf)
    for _ in range(6):
        D = oracle.srgemm("minimum", "plus", D, D, D, np.float16(0), np.float16(0), inf)
    assert np.array_equal(D.astype(np.float64), want)


def test_int8_operands_are_widened_first(oracle):
    """int8 A and B with int32 C, D, scalars and accumulator: every pair against numpy on int64 (no value here
    leaves the int32 range), both loops, all layouts."""
    rng = np.random.default_rng(3)
    m, n, k = 19, 23, 41
    for la, lb, lc in itertools.product("FC", repeat=3):
        A = np.asarray(rng.integers(-128, 128, (m, k)).astype(np.int8), order=la)
        B = np.asarray(rng.integers(-128, 128, (k, n)).astype(np.int8), order=lb)
        C = np.asarray(rng.integers(-10 ** 6, 10 ** 6, (m, n)).astype(np.int32), order=lc)
        a, b, c = A.astype(np.int64), B.astype(np.int64), C.astype(np.int64)
        sums = a[:, :, None] + b[None, :, :]
        wants = {("plus", "multiplies"): (7 * (a @ b) - 3 * c, 7, -3, 0),
                 ("minimum", "plus"): (np.minimum(sums.min(1) + 5, c + 2), 5, 2, 2 ** 31 - 1),
                 ("maximum", "plus"): (np.maximum(sums.max(1), c), 0, 0, -2 ** 31),
                 ("maximum", "minimum"): (np.maximum(np.minimum(np.minimum(a[:, :, None], b[None, :, :]).max(1), 100), np.minimum(c, 50)),
                                          100, 50, -2 ** 31),
                 ("bit_xor", "bit_and"): (np.bitwise_xor.reduce(a[:, :, None] & b[None, :, :], axis=1) ^ c, -1, -1, 0)}
        for (add, mult), (want, alpha, beta, ident) in wants.items():
            for naive in (False, True):
                got = oracle.srgemm(add, mult, A, B, C, alpha, beta, ident, naive=naive)
                assert np.array_equal(got.astype(np.int64), want), (add, mult, la, lb, lc, naive)


def test_blocked_equals_naive_on_ragged_and_submatrix(oracle):
    big_a = inputs.uniform(1, 140, 90)
    big_b = inputs.uniform(2, 90, 150)
    big_c = inputs.uniform(3, 140, 150)
    for (r0, c0, m, n, k) in [(0, 0, 125, 125, 80), (15, 21, 70, 65, 33), (3, 2, 97, 130, 90)]:
        A, B, C = big_a[r0:r0 + m, :k], big_b[:k, c0:c0 + n], big_c[r0:r0 + m, c0:c0 + n]  # ld > extent
        for add, mult, ident in [("minimum", "plus", np.inf), ("maximum", "minimum", -np.inf), ("plus", "multiplies", 0.0)]:
            one = {"plus": 0.0, "minimum": np.inf, "multiplies": 1.0}[mult]
            x = oracle.srgemm(add, mult, A, B, C, one, one, ident, naive=False, nthreads=3)
            y = oracle.srgemm(add, mult, A, B, C, one, one, ident, naive=True)
            assert bits(x) == bits(y)


def test_plus_times_is_gemm(oracle):
    A = inputs.integers(1, 40, 50, -8, 8, np.float32)
    B = inputs.integers(2, 50, 30, -8, 8, np.float32)
    C = inputs.integers(3, 40, 30, -8, 8, np.float32)
    got = oracle.srgemm("plus", "multiplies", A, B, C, 2.0, 3.0, 0.0)
    want = 2.0 * (A.astype(np.float64) @ B.astype(np.float64)) + 3.0 * C
    assert np.array_equal(got.astype(np.float64), want)  # small integers: exact in fp32
    An, Bn = inputs.normal(4, 64, 300, np.float64), inputs.normal(5, 300, 48, np.float64)
    got = oracle.srgemm("plus", "multiplies", An, Bn, np.zeros((64, 48), order="F"), 1.0, 0.0, 0.0)
    bound = 1e-12 * (np.abs(An) @ np.abs(Bn))
    assert np.all(np.abs(got - An @ Bn) <= bound)


def test_gf2_and_boolean_closed_forms(oracle):
    A = inputs.bernoulli(1, 45, 60, 0.3)
    B = inputs.bernoulli(2, 60, 38, 0.3)
    Z = np.zeros((45, 38), dtype=np.int32, order="F")
    prod = A.astype(np.int64) @ B.astype(np.int64)
    got = oracle.srgemm("bit_xor", "logical_and", A, B, Z, 1, 0, 0)
    assert np.array_equal(got, (prod % 2).astype(np.int32))
    got = oracle.srgemm("logical_or", "logical_and", A, B, Z, 1, 0, 0)
    assert np.array_equal(got, (prod > 0).astype(np.int32))
    # logical_and is not bitwise: 6 && 9 = 1, 6 & 9 = 0  (functional.h:212)
    six, nine = np.full((1, 1), 6, np.int32), np.full((1, 1), 9, np.int32)
    z1 = np.zeros((1, 1), np.int32)
    assert oracle.srgemm("bit_xor", "logical_and", six, nine, z1, 1, 0, 0)[0, 0] == 1
    assert oracle.srgemm("bit_xor", "bit_and", six, nine, z1, -1, 0, 0)[0, 0] == 0
    # bit-packed GF(2): 32 independent products, one per bit plane
    Aw, Bw = inputs.words32(3, 20, 37), inputs.words32(4, 37, 25)
    Zw = np.zeros((20, 25), dtype=np.uint32, order="F")
    got = oracle.srgemm("bit_xor", "bit_and", Aw, Bw, Zw, 0xFFFFFFFF, 0, 0)
    for b in (0, 7, 31):
        pa, pb = ((Aw >> np.uint32(b)) & 1).astype(np.int64), ((Bw >> np.uint32(b)) & 1).astype(np.int64)
        assert np.array_equal((got >> np.uint32(b)) & 1, ((pa @ pb) % 2).astype(np.uint32))


def floyd_warshall(D):
    D = D.astype(np.float64).copy()
    for kk in range(D.shape[0]):
        D = np.minimum(D, D[:, kk:kk + 1] + D[kk:kk + 1, :])
    return D


def test_minplus_closure_is_floyd_warshall(oracle):
    n = 48
    D = inputs.graph_distances(9, n, density=0.15, integer_weights=True)  # sums < 2^24: exact in fp32
    cur = D
    for _ in range(6):  # 2^6 >= n - 1
        cur = oracle.srgemm("minimum", "plus", cur, cur, cur, 0.0, 0.0, np.inf)
    assert np.array_equal(cur.astype(np.float64), floyd_warshall(D))
    again = oracle.srgemm("minimum", "plus", cur, cur, cur, 0.0, 0.0, np.inf)
    assert bits(again) == bits(cur)  # closed: idempotent


def test_maxmin_closure_is_widest_path(oracle):
    n = 24
    W = inputs.uniform(3, n, n, 0.0, 1.0, np.float64)
    np.fill_diagonal(W, np.inf)
    cur = W
    for _ in range(5):
        cur = oracle.srgemm("maximum", "minimum", cur, cur, cur, np.inf, np.inf, -np.inf)
    ref = W.copy()
    for kk in range(n):
        ref = np.maximum(ref, np.minimum(ref[:, kk:kk + 1], ref[kk:kk + 1, :]))
    assert np.array_equal(cur, ref)


def test_invariants(oracle):
    m, n, k = 37, 29, 41
    A, B, C = inputs.uniform(1, m, k), inputs.uniform(2, k, n), inputs.uniform(3, m, n)
    inf = np.float32(np.inf)
    base = oracle.srgemm("minimum", "plus", A, B, C, 0.0, inf, inf)
    # beta = semiring zero: D does not depend on C
    other = oracle.srgemm("minimum", "plus", A, B, inputs.uniform(4, m, n), 0.0, inf, inf)
    assert bits(base) == bits(other)
    # beta = semiring one: D = min(A (x) B, C)
    withc = oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, inf)
    assert np.array_equal(withc, np.minimum(base, C))
    # A (x) I = A, I = semiring one on the diagonal, zero elsewhere
    eye = np.full((k, k), inf, dtype=np.float32, order="F")
    np.fill_diagonal(eye, 0.0)
    assert np.array_equal(oracle.srgemm("minimum", "plus", A, eye, np.zeros((m, k), np.float32, order="F"), 0.0, inf, inf), A)
    # order-freeness: permuting k changes nothing (the basis of bit-exact parity)
    perm = np.argsort(inputs.uniform(8, k, 1)[:, 0])
    assert bits(oracle.srgemm("minimum", "plus", np.asfortranarray(A[:, perm]), np.asfortranarray(B[perm, :]), C, 0.0, inf, inf)) == bits(base)
    # transposition: (A (x) B)^T = B^T (x) A^T
    tr = oracle.srgemm("minimum", "plus", np.asfortranarray(B.T), np.asfortranarray(A.T), np.asfortranarray(C.T), 0.0, inf, inf)
    assert np.array_equal(tr.T, base)
    # every layout combination gives the same values
    for la, lb, lc in itertools.product("FC", repeat=3):
        got = oracle.srgemm("minimum", "plus", np.asarray(A, order=la), np.asarray(B, order=lb), np.asarray(C, order=lc), 0.0, 0.0, inf)
        assert np.array_equal(got, withc)
    # reference-valued identity (numeric_limits::max) behaves like +inf on this data
    fmax = np.finfo(np.float32).max
    assert np.array_equal(oracle.srgemm("minimum", "plus", A, B, C, 0.0, fmax, fmax), base)


@pytest.mark.parametrize("slices", [1, 2, 3, 8, 16])
def test_splitk_model(oracle, slices):
    m, n, k = 40, 24, 200
    A, B, C = inputs.uniform(1, m, k, 0, 10), inputs.uniform(2, k, n, 0, 10), inputs.uniform(3, m, n, 0, 10)
    inf = np.float32(np.inf)
    for beta in (inf, np.float32(0.0)):  # zero (no source) and one
        want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, beta, inf)
        got = oracle.srgemm_splitk("minimum", "plus", A, B, C, 0.0, beta, inf, 0.0, slices)
        assert bits(got) == bits(want)  # the reference example's own check (splitk_srgemm.cu:270-287)
    # plus-times: slicing changes the summation order, not the value on small integers
    Ai, Bi = inputs.integers(4, m, k, -8, 8), inputs.integers(5, k, n, -8, 8)
    want = oracle.srgemm("plus", "multiplies", Ai, Bi, C, 1.0, 0.0, 0.0)
    got = oracle.srgemm_splitk("plus", "multiplies", Ai, Bi, C, 1.0, 0.0, 0.0, 1.0, slices)
    assert bits(got) == bits(want)


def literal_serial_splitk(add, mult, A, B, C, alpha, beta, ident, one, slices, tbk=8):
    """The serial split-K as the reference's workgroups perform it, in Python scalars: slice z
    covers k in [z*ks, min(K, (z+1)*ks)) with ks = ceil(ceil(K/tbk)/slices)*tbk
    (kernel/srgemm.h:97-100, :184-189); its epilogue reads C (z = 0) or D (z > 0, beta replaced
    by the multiplicative identity) and writes D (kernel/srgemm.h:290-300,
    semiring_linear_combination.h:129-134); an unneeded source drops the add (:166-183)."""
    f_add, f_mul = PY_OPS[add], PY_OPS[mult]
    t = A.dtype.type
    m, k = A.shape
    n = B.shape[1]
    ks = -(-(-(-k // tbk)) // slices) * tbk
    D = np.zeros((m, n), dtype=A.dtype)
    with np.errstate(over="ignore", invalid="ignore"):
        for z in range(slices):
            b = t(beta) if z == 0 else t(one)
            need = t(ident) != t(f_mul(b, t(one)))
            for i in range(m):
                for j in range(n):
                    acc = t(ident)
                    for kk in range(min(k, z * ks), min(k, (z + 1) * ks)):
                        acc = t(f_add(t(f_mul(A[i, kk], B[kk, j])), acc))
                    lhs = t(f_mul(t(alpha), acc))
                    src = C[i, j] if z == 0 else D[i, j]
                    D[i, j] = t(f_add(lhs, t(f_mul(b, src)))) if need else lhs
    return D


@pytest.mark.parametrize("slices", [1, 2, 3, 5, 8])
def test_serial_splitk_model_against_literal_chain(oracle, slices):
    m, n, k = 9, 7, 61
    inf = np.float32(np.inf)
    A, B, C = inputs.uniform(11, m, k, -2, 2), inputs.uniform(12, k, n, -2, 2), inputs.uniform(13, m, n, -2, 2)
    cases = [
        ("minimum", "plus", 0.25, 0.0, inf, 0.0),          # beta = one: C joins the chain
        ("minimum", "plus", 0.25, inf, inf, 0.0),          # beta = zero: C is not read
        ("plus", "multiplies", 1.5, -0.75, 0.0, 1.0),      # rounding depends on the slice boundaries
        ("minimum", "multiplies", -2.0, 1.0, inf, 1.0),    # alpha < 0: alpha per partial differs from alpha on the total
        ("maximum", "minimum", 1.0, 0.5, -inf, inf),
    ]
    for add, mult, alpha, beta, ident, one in cases:
        want = literal_serial_splitk(add, mult, A, B, C, alpha, beta, ident, one, slices)
        got = oracle.srgemm_splitk_serial(add, mult, A, B, C, alpha, beta, ident, one, slices)
        assert bits(got) == bits(want), (add, mult, slices)
    Au, Bu, Cu = inputs.words32(14, m, k), inputs.words32(15, k, n), inputs.words32(16, m, n)
    full = np.uint32(0xFFFFFFFF)
    want = literal_serial_splitk("bit_xor", "bit_and", Au, Bu, Cu, full, full, 0, full, slices)
    got = oracle.srgemm_splitk_serial("bit_xor", "bit_and", Au, Bu, Cu, full, full, 0, full, slices)
    assert bits(got) == bits(want)


def test_serial_splitk_model_invariants(oracle):
    m, n, k = 40, 24, 200
    inf = np.float32(np.inf)
    A, B, C = inputs.uniform(1, m, k, 0, 10), inputs.uniform(2, k, n, 0, 10), inputs.uniform(3, m, n, 0, 10)
    for slices in (1, 2, 3, 8, 16, 40):  # 40 > K/8: trailing slices have no k range
        for beta in (inf, np.float32(0.0)):
            # an idempotent, order-free add: the chain equals the unsplit product bit for bit
            want = oracle.srgemm("minimum", "plus", A, B, C, 0.0, beta, inf)
            got = oracle.srgemm_splitk_serial("minimum", "plus", A, B, C, 0.0, beta, inf, 0.0, slices)
            assert bits(got) == bits(want)
        # an unneeded source is never read: NaN in C must not reach D (the host reference would propagate it)
        Cn = np.full_like(C, np.nan)
        got = oracle.srgemm_splitk_serial("minimum", "plus", A, B, Cn, 0.0, inf, inf, 0.0, slices)
        assert bits(got) == bits(oracle.srgemm("minimum", "plus", A, B, C, 0.0, inf, inf))
        # D may alias C
        Cc = C.copy()
        oracle.srgemm_splitk_serial("minimum", "plus", A, B, Cc, 0.0, 0.0, inf, 0.0, slices, out=Cc)
        assert bits(Cc) == bits(oracle.srgemm("minimum", "plus", A, B, C, 0.0, 0.0, inf))
    # plus-times on small integers is exact whatever the slicing; alpha multiplies every partial, beta only C
    Ai, Bi, Ci = inputs.integers(4, m, k, -8, 8), inputs.integers(5, k, n, -8, 8), inputs.integers(6, m, n, -8, 8)
    want = oracle.srgemm("plus", "multiplies", Ai, Bi, Ci, 2.0, -3.0, 0.0)
    for slices in (2, 7):
        got = oracle.srgemm_splitk_serial("plus", "multiplies", Ai, Bi, Ci, 2.0, -3.0, 0.0, 1.0, slices)
        assert bits(got) == bits(want)


# ---- min-plus product with predecessor tracking (test/regress/include/fwgpu/cpu_srgemm.hpp:20-48) ----

def fw_inputs(seed, m, n, k, dtype, ties=True):
    """Small-integer weights (many equal products), some +inf, leading dimensions larger than the extents."""
    rng = np.random.default_rng(seed)
    def mat(r, c, lo, hi, pad):
        buf = np.full((r + pad, c), np.nan, dtype=dtype, order="F")
        v = rng.integers(lo, hi, (r, c)).astype(dtype) if ties else rng.random((r, c)).astype(dtype) * 10
        v[rng.random((r, c)) < 0.2] = np.inf
        buf[:r] = v
        return buf[:r]
    A, B = mat(m, k, 0, 6, 3), mat(k, n, 0, 6, 1)
    dist = mat(m, n, 2, 9, 2)
    parent = np.full((m + 5, n), -7, dtype=np.int32, order="F")[:m]
    return A, B, dist, parent


def fw_expected(A, B, dist, parent):
    """Independent statement: the smallest product, where it first occurs (numpy's argmin returns the
    first occurrence), taken only when strictly smaller than the old distance."""
    prods = A[:, :, None] + B[None, :, :]              # m x k x n
    best = prods.min(axis=1) if A.shape[1] else np.full(dist.shape, np.inf, dist.dtype)
    where = prods.argmin(axis=1) if A.shape[1] else np.zeros(dist.shape, np.int64)
    better = best < dist
    return np.where(better, best, dist), np.where(better, where, parent).astype(np.int32)


def test_fwgemm_hand_worked_graph(oracle):
    inf = np.inf
    D = np.asfortranarray(np.array([[0, 1, inf], [inf, 0, 2], [1, inf, 0]], dtype=np.float32))
    dist, parent = D.copy(order="F"), np.full((3, 3), -1, np.int32, order="F")
    oracle.fwgemm(D, D, dist, parent)
    # 0 -> 2 through 1 (1 + 2), 1 -> 0 through 2 (2 + 1), 2 -> 1 through 0 (1 + 1)
    assert dist.tolist() == [[0, 1, 3], [3, 0, 2], [1, 2, 0]]
    assert parent.tolist() == [[-1, -1, 1], [2, -1, -1], [-1, 0, -1]]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("shape", [(1, 1, 1), (5, 7, 3), (33, 20, 41), (64, 64, 64), (3, 2, 0)])
def test_fwgemm_first_strict_minimum(oracle, dtype, shape):
    for ties in (True, False):
        A, B, dist, parent = fw_inputs(shape[0] * 7 + shape[2], *shape, dtype, ties)
        want_d, want_p = fw_expected(A, B, dist, parent)
        got_d, got_p = dist.copy(order="F"), parent.copy(order="F")
        oracle.fwgemm(A, B, got_d, got_p)
        assert_same_bits(got_d, want_d.astype(dtype), "dist")
        assert np.array_equal(got_p, want_p)
        # dist is the min-plus SRGEMM with the old distances as C
        if shape[2] > 0:
            srgemm = oracle.srgemm("minimum", "plus", A, B, dist, 0.0, 0.0, np.inf)
            assert_same_bits(got_d, srgemm, "dist vs srgemm")
        if ties and min(shape) > 4:
            assert (want_p == -7).any() and (want_p >= 0).any()   # both branches were taken


def expand_path(parent, i, j):
    """Vertices strictly between i and j on the path the parent matrix encodes."""
    k = parent[i, j]
    if k < 0:
        return []
    return expand_path(parent, i, k) + [int(k)] + expand_path(parent, k, j)


def test_fwgemm_squaring_gives_shortest_paths(oracle):
    from scipy.sparse.csgraph import floyd_warshall as scipy_fw
    rng = np.random.default_rng(11)
    n = 48
    W = np.where(rng.random((n, n)) < 0.15, rng.integers(1, 20, (n, n)), np.inf).astype(np.float32)
    np.fill_diagonal(W, 0)
    dist, parent = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    for _ in range(6):                                      # 2^6 >= n - 1 edges
        snap = dist.copy(order="F")
        oracle.fwgemm(snap, snap, dist, parent)
    assert np.array_equal(dist.astype(np.float64), scipy_fw(W.astype(np.float64)))
    for i in range(n):
        for j in range(n):
            if i == j or np.isinf(dist[i, j]):
                assert parent[i, j] == -1
                continue
            hops = [i] + expand_path(parent, i, j) + [j]
            assert all(np.isfinite(W[a, b]) for a, b in zip(hops, hops[1:]))    # every hop is an edge
            assert sum(W[a, b] for a, b in zip(hops, hops[1:])) == dist[i, j]   # and the path has that length


# ---- blocked Floyd-Warshall (oracle/host_blocked_fw.c) -------------------------------------

def literal_floyd_warshall(W):
    """The textbook triple loop, k outermost, with the intermediate vertex as predecessor."""
    n = W.shape[0]
    d, p = W.copy(), np.full((n, n), -1, np.int32)
    for k in range(n):
        cand = d[:, k:k + 1] + d[k:k + 1, :]
        better = cand < d
        d[better], p[better] = cand[better], k
    return d, p


def test_blocked_fw_hand_worked_graph(oracle):
    inf = np.inf
    # 0 -> 1 -> 2 -> 3 is a chain of unit edges, 0 -> 3 costs 10 directly
    W = np.array([[0, 1, inf, 10], [inf, 0, 1, inf], [inf, inf, 0, 1], [inf, inf, inf, 0]], dtype=np.float32)
    for block in (1, 2, 3, 4, 128):
        dist, parent = np.asfortranarray(W), np.full((4, 4), -1, np.int32, order="F")
        oracle.apsp_blocked(dist, parent, block)
        assert dist.tolist() == [[0, 1, 2, 3], [inf, 0, 1, 2], [inf, inf, 0, 1], [inf, inf, inf, 0]], block
        assert [0] + expand_path(parent, 0, 3) + [3] == [0, 1, 2, 3], block
        assert parent[0, 1] == -1 and parent[3, 0] == -1


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("n,block", [(1, 4), (7, 3), (31, 8), (50, 16), (96, 32), (130, 128), (150, 64)])
def test_blocked_fw_on_integer_weights(oracle, n, block, dtype):
    """Integer weights: every order of additions is exact, so the distances equal scipy's
    Floyd-Warshall and the textbook loop's; parents need not (ties), but must describe paths
    of exactly the distance."""
    from scipy.sparse.csgraph import floyd_warshall as scipy_fw
    rng = np.random.default_rng(1000 * n + block)
    W = np.where(rng.random((n, n)) < max(0.05, 2.5 / n), rng.integers(1, 30, (n, n)), np.inf).astype(dtype)
    np.fill_diagonal(W, 0)
    dist, parent = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    oracle.apsp_blocked(dist, parent, block)
    assert np.array_equal(dist.astype(np.float64), scipy_fw(W.astype(np.float64)))
    assert np.array_equal(dist, literal_floyd_warshall(W)[0])
    for i in range(n):
        for j in range(n):
            if i == j or np.isinf(dist[i, j]):
                assert parent[i, j] == -1
                continue
            hops = [i] + expand_path(parent, i, j) + [j]
            assert all(np.isfinite(W[a, b]) for a, b in zip(hops, hops[1:]))
            assert sum(W[a, b] for a, b in zip(hops, hops[1:])) == dist[i, j]


def test_blocked_fw_with_one_block_is_the_textbook_loop(oracle):
    """A block as large as the matrix leaves the in-block loop (the products that follow find
    nothing to improve on exact sums): distances and parents of the textbook algorithm."""
    rng = np.random.default_rng(3)
    n = 40
    W = np.where(rng.random((n, n)) < 0.2, rng.integers(1, 12, (n, n)), np.inf).astype(np.float32)
    np.fill_diagonal(W, 0)
    dist, parent = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    oracle.apsp_blocked(dist, parent, n)
    want_d, want_p = literal_floyd_warshall(W)
    assert np.array_equal(dist, want_d) and np.array_equal(parent, want_p)


def test_blocked_fw_leading_dimensions(oracle):
    rng = np.random.default_rng(4)
    n = 37
    W = np.where(rng.random((n, n)) < 0.2, rng.integers(1, 9, (n, n)), np.inf).astype(np.float64)
    np.fill_diagonal(W, 0)
    big = np.full((n + 5, n), -3.0, order="F")
    big[:n] = W
    pbig = np.full((n + 2, n), -9, np.int32, order="F")
    pbig[:n] = -1
    oracle.apsp_blocked(big[:n], pbig[:n], 16)
    dist, parent = np.asfortranarray(W), np.full((n, n), -1, np.int32, order="F")
    oracle.apsp_blocked(dist, parent, 16)
    assert np.array_equal(big[:n], dist) and np.array_equal(pbig[:n], parent)
    assert (big[n:] == -3.0).all() and (pbig[n:] == -9).all()


# ---- the C++ split-K models that check the kernels built from user functors ----------------------------------

@pytest.mark.parametrize("form", ["parallel", "serial"])
@pytest.mark.parametrize("pair", ["plustimes", "mintimes"])
def test_cpp_splitk_models_agree_with_the_c_oracle(oracle, form, pair):
    """oracle/include/cuasr/reference/srgemm/host_srgemm_splitk.h restates, for any functor pair, the two split-K
    models that oracle/host_srgemm.c holds for the library's operators (pinned above against literal Python
    chains).  On floating-point plus-times with non-integer data, and on min-times under a negative alpha, the
    bits depend on where a slice ends and on the order of the fold, so agreement pins both."""
    import subprocess
    import build_cpp
    binary = build_cpp.build("host_splitk_models")
    add, mult, alpha, beta, ident = ("plus", "multiplies", 1.25, 0.5, 0.0) if pair == "plustimes" else ("minimum", "multiplies", -1.5, 1.0, np.finfo(np.float32).max)
    value = lambda seed, count: (((np.arange(count, dtype=np.uint32) * 37 + seed * 11 + (np.arange(count, dtype=np.uint32) >> 3) * 5) % 101).astype(np.float32) / np.float32(7) - np.float32(3))
    differs = 0
    for m, n, k, slices in [(3, 2, 20, 2), (5, 7, 100, 3), (4, 6, 77, 8), (9, 3, 301, 5), (2, 2, 7, 4), (6, 5, 64, 1)]:
        out = subprocess.run([binary, form, pair, str(m), str(n), str(k), str(slices)], capture_output=True, text=True, check=True).stdout.split()
        got = np.array([int(x, 16) for x in out], dtype=np.uint32).view(np.float32).reshape(n, m).T    # column-major m x n
        A = value(1, m * k).reshape(k, m).T            # column-major m x k
        B = value(2, k * n).reshape(k, n)              # row-major k x n
        C = np.asfortranarray(value(3, m * n).reshape(n, m).T)
        model = oracle.srgemm_splitk if form == "parallel" else oracle.srgemm_splitk_serial
        want = model(add, mult, np.asfortranarray(A), np.ascontiguousarray(B), C, alpha, beta, ident, 1.0, slices, tbk=8)
        assert_same_bits(np.ascontiguousarray(got), np.ascontiguousarray(want), f"{form} {pair} {m}x{n}x{k} S={slices}")
        plain = oracle.srgemm(add, mult, np.asfortranarray(A), np.ascontiguousarray(B), C, alpha, beta, ident)
        differs += int(np.ascontiguousarray(plain).tobytes() != np.ascontiguousarray(want).tobytes())
    # (the parallel form folds raw minima and scales once: with an order-free add it cannot differ from the unsplit
    # result, whatever the slices -- which the assertion above has just shown for the C++ model)
    if not (pair == "mintimes" and form == "parallel"):
        assert differs >= 2, "cases whose split-K result equals the unsplit one pin nothing about the slices"
