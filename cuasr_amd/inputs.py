"""Seeded synthetic inputs for the SRGEMM workloads.

A counter-based generator (splitmix64 finaliser over ``seed + index``) so the
same matrix can be produced anywhere, in any order, with numpy alone; no
library-specific distribution code is involved.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed, count, offset=0):
    """``count`` 64-bit words: word i is mix(seed*G + (offset+i+1)*G).  (So seed s + 1 gives the stream of
    seed s moved on by one word: matrices that must be unrelated take seeds further apart than their size.)"""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + count + 1, dtype=np.uint64)
        z = (np.uint64(seed) * _GOLDEN + np.uint64(0x632BE59BD9B4E019)) + idx * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        z = z ^ (z >> np.uint64(31))
    return z


def _unit(seed, count, dtype):
    """Uniform [0, 1): top 24 bits (float32) or top 53 bits (float64)."""
    bits = splitmix64(seed, count)
    if np.dtype(dtype) == np.float32:
        return ((bits >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24))
    return (bits >> np.uint64(11)).astype(np.float64) * (2.0 ** -53)


def _shape(values, rows, cols, order):
    # values are generated in column-major element order regardless of the
    # storage order, so a matrix has the same entries in either layout
    return np.asarray(values.reshape((cols, rows)).T, order=order)


def uniform(seed, rows, cols, lo=0.0, hi=1.0, dtype=np.float32, order="F"):
    """rows x cols matrix, entries lo + (hi-lo)*u, u uniform in [0, 1)."""
    dtype = np.dtype(dtype)
    u = _unit(seed, rows * cols, dtype)
    vals = (dtype.type(lo) + dtype.type(hi - lo) * u).astype(dtype)
    return _shape(vals, rows, cols, order)


def integers(seed, rows, cols, lo, hi, dtype=np.float32, order="F"):
    """Integer-valued entries uniform in [lo, hi] (inclusive)."""
    bits = splitmix64(seed, rows * cols)
    span = np.uint64(hi - lo + 1)
    vals = ((bits >> np.uint64(33)) % span).astype(np.int64) + lo
    return _shape(vals.astype(dtype), rows, cols, order)


def words32(seed, rows, cols, order="F"):
    """Uniform 32-bit words (bit-packed GF(2) operands)."""
    bits = splitmix64(seed, rows * cols)
    return _shape((bits >> np.uint64(32)).astype(np.uint32), rows, cols, order)


def bernoulli(seed, rows, cols, p, dtype=np.int32, order="F"):
    """0/1 entries, 1 with probability p."""
    u = _unit(seed, rows * cols, np.float64)
    return _shape((u < p).astype(dtype), rows, cols, order)


def normal(seed, rows, cols, dtype=np.float32, order="F"):
    """Standard normal by Box-Muller on two generator streams."""
    count = rows * cols
    u1 = _unit(seed, count, np.float64)
    u2 = _unit(seed ^ 0x5DEECE66D, count, np.float64)
    r = np.sqrt(-2.0 * np.log(1.0 - u1))
    vals = (r * np.cos(2.0 * np.pi * u2)).astype(dtype)
    return _shape(vals, rows, cols, order)


def graph_distances(seed, n, density=0.10, lo=1.0, hi=100.0, dtype=np.float32,
                    order="F", integer_weights=False):
    """Directed-graph distance matrix: 0 on the diagonal, an edge with
    probability ``density`` weighted uniform [lo, hi), +inf elsewhere."""
    dtype = np.dtype(dtype)
    pick = _unit(seed, n * n, np.float64)
    w = _unit(seed + 1, n * n, dtype)
    vals = (dtype.type(lo) + dtype.type(hi - lo) * w).astype(dtype)
    if integer_weights:
        vals = np.floor(vals).astype(dtype)
    vals = np.where(pick < density, vals, dtype.type(np.inf)).astype(dtype)
    d = _shape(vals, n, n, order)
    np.fill_diagonal(d, 0)
    return d
