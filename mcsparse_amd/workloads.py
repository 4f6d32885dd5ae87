"""Seeded synthetic CSR matrices for the benchmark configurations, as numpy arrays.

All generators are vectorised numpy driven by numpy's PCG64 (bit-reproducible across
machines for the calls used here), return int32 row offsets / column indices with sorted,
distinct columns per row, and take the index base (0 or 1) as a parameter.
"""
import numpy as np

SEED0 = 0x5EED0000


class Csr:
    """Host-side CSR matrix: ptr[m+1], col[nnz], val[nnz] (index base included in ptr/col)."""

    def __init__(self, m, n, ptr, col, val, base=0):
        self.m, self.n, self.base = int(m), int(n), int(base)
        self.ptr = np.ascontiguousarray(ptr, dtype=np.int32)
        self.col = np.ascontiguousarray(col, dtype=np.int32)
        self.val = np.ascontiguousarray(val)
        self.nnz = int(self.col.shape[0])

    def with_base(self, base):
        d = int(base) - self.base
        return Csr(self.m, self.n, self.ptr + d, self.col + d, self.val, base)

    def to_scipy(self):
        import scipy.sparse as sp
        return sp.csr_matrix((self.val, self.col - self.base, self.ptr - self.base), shape=(self.m, self.n))

    def row_lengths(self):
        return np.diff(self.ptr.astype(np.int64))


def _rng(config_id, stream=0):
    return np.random.Generator(np.random.PCG64([SEED0 + config_id, stream]))


def _uniform_pm1(rng, size, dtype):
    return (2.0 * rng.random(size) - 1.0).astype(dtype)


def laplacian_5pt(grid=256, dtype=np.float32, base=0):
    """Config 1: 5-point Laplacian on a grid x grid mesh, row-major numbering, 4 / -1."""
    g = int(grid)
    idx = np.arange(g * g, dtype=np.int64)
    iy, ix = idx // g, idx % g
    cols = np.stack([idx - g, idx - 1, idx, idx + 1, idx + g], axis=1)
    keep = np.stack([iy > 0, ix > 0, np.ones_like(ix, bool), ix < g - 1, iy < g - 1], axis=1)
    vals = np.broadcast_to(np.array([-1, -1, 4, -1, -1], dtype=dtype), cols.shape)
    ptr = np.concatenate([[0], np.cumsum(keep.sum(axis=1))])
    return Csr(g * g, g * g, ptr + base, cols[keep] + base, vals[keep], base)


def uniform_rows(m=1 << 20, n=None, per_row=16, dtype=np.float64, base=0, config_id=2):
    """Config 2: exactly per_row distinct, sorted, uniformly drawn columns per row; N(0,1) values."""
    n = m if n is None else n
    rng = _rng(config_id)
    # sorted draws from [0, n - per_row] plus 0..per_row-1 are strictly increasing and stay below n
    d = np.sort(rng.integers(0, n - per_row + 1, size=(m, per_row), dtype=np.int64), axis=1)
    col = d + np.arange(per_row, dtype=np.int64)[None, :]
    val = rng.standard_normal(size=m * per_row).astype(dtype)
    ptr = np.arange(m + 1, dtype=np.int64) * per_row
    return Csr(m, n, ptr + base, col.reshape(-1) + base, val, base)


def mixed_rows(m=1 << 20, n=None, per_row=16, long_rows=64, long_len=100_000, dtype=np.float32, base=0, config_id=6):
    """Mostly short rows plus a handful of very long ones, spread evenly over the matrix: what a row-length-binned
    dispatch is for.  Short rows as in uniform_rows; a long row holds long_len distinct sorted columns."""
    n = m if n is None else n
    rng = _rng(config_id)
    lengths = np.full(m, per_row, dtype=np.int64)
    where = (np.arange(long_rows, dtype=np.int64) * m) // max(long_rows, 1) + m // (2 * max(long_rows, 1))
    lengths[where] = min(long_len, n)
    ptr = np.concatenate([[0], np.cumsum(lengths)])
    col = np.empty(int(ptr[-1]), dtype=np.int64)
    short = np.ones(m, dtype=bool)
    short[where] = False
    d = np.sort(rng.integers(0, n - per_row + 1, size=(int(short.sum()), per_row), dtype=np.int64), axis=1)
    d += np.arange(per_row, dtype=np.int64)[None, :]
    starts = ptr[:-1][short]
    col[(starts[:, None] + np.arange(per_row, dtype=np.int64)[None, :]).reshape(-1)] = d.reshape(-1)
    for r in where:
        col[ptr[r]:ptr[r + 1]] = np.sort(rng.choice(n, size=int(lengths[r]), replace=False))
    val = _uniform_pm1(rng, int(ptr[-1]), dtype)
    return Csr(m, n, ptr + base, col + base, val, base)


def zipf_row_lengths(m, exponent=1.8, max_len=200_000, rng=None):
    """Row lengths with pmf proportional to k^-exponent on [1, max_len] (inverse CDF)."""
    k = np.arange(1, max_len + 1, dtype=np.float64)
    cdf = np.cumsum(k ** (-exponent))
    cdf /= cdf[-1]
    u = rng.random(m)
    return (np.searchsorted(cdf, u, side="left") + 1).astype(np.int64)


def power_law(m=1 << 22, n=None, exponent=1.8, max_len=200_000, dtype=np.float32, base=0, config_id=3):
    """Config 3: Zipf(exponent) row lengths clipped at max_len (and at n), uniform sorted distinct
    columns, U[-1,1] values."""
    n = m if n is None else n
    rng = _rng(config_id)
    lens = np.minimum(zipf_row_lengths(m, exponent, min(max_len, n), rng), n)
    ptr = np.concatenate([[0], np.cumsum(lens)])
    nnz = int(ptr[-1])
    row_of = np.repeat(np.arange(m, dtype=np.int64), lens)
    pos_in_row = np.arange(nnz, dtype=np.int64) - ptr[row_of]
    # d sorted inside each row, then + position: strictly increasing columns below n
    span = (n - lens + 1)[row_of]
    d = (rng.random(nnz) * span).astype(np.int64)
    np.minimum(d, span - 1, out=d)
    key = np.sort((row_of << 32) | d)
    col = (key & 0xFFFFFFFF) + pos_in_row
    val = _uniform_pm1(rng, nnz, dtype)
    return Csr(m, n, ptr + base, col + base, val, base)


def stencil_27pt(grid=128, dtype=np.float32, base=0, config_id=4):
    """Config 4: 27-point stencil on a grid^3 mesh, lexicographic numbering, U[-1,1] values."""
    g = int(grid)
    rng = _rng(config_id)
    idx = np.arange(g ** 3, dtype=np.int64)
    iz, iy, ix = idx // (g * g), (idx // g) % g, idx % g
    cols, keep = [], []
    for dz in (-1, 0, 1):
        for dy in (-1, 0, 1):
            for dx in (-1, 0, 1):
                cols.append(idx + dz * g * g + dy * g + dx)
                keep.append((iz + dz >= 0) & (iz + dz < g) & (iy + dy >= 0) & (iy + dy < g) & (ix + dx >= 0) &
                            (ix + dx < g))
    cols = np.stack(cols, axis=1)
    keep = np.stack(keep, axis=1)
    ptr = np.concatenate([[0], np.cumsum(keep.sum(axis=1))])
    col = cols[keep]
    val = _uniform_pm1(rng, col.shape[0], dtype)
    return Csr(g ** 3, g ** 3, ptr + base, col + base, val, base)


def random_ragged(m, n, mean_len, dtype=np.float32, base=0, seed=0, empty_fraction=0.2):
    """Small test matrix with empty rows and ragged lengths (not a benchmark configuration)."""
    rng = np.random.Generator(np.random.PCG64([SEED0 + 99, seed]))
    lens = rng.poisson(mean_len, size=m).astype(np.int64)
    lens[rng.random(m) < empty_fraction] = 0
    lens = np.minimum(lens, n)
    ptr = np.concatenate([[0], np.cumsum(lens)])
    nnz = int(ptr[-1])
    row_of = np.repeat(np.arange(m, dtype=np.int64), lens)
    pos_in_row = np.arange(nnz, dtype=np.int64) - ptr[row_of]
    span = (n - lens + 1)[row_of]
    d = np.minimum((rng.random(nnz) * span).astype(np.int64), span - 1)
    key = np.sort((row_of << 32) | d)
    col = (key & 0xFFFFFFFF) + pos_in_row
    val = _uniform_pm1(rng, nnz, dtype)
    return Csr(m, n, ptr + base, col + base, val, base)


def dense_vector(size, dtype, config_id, stream):
    return _uniform_pm1(_rng(config_id, stream), size, dtype)


def spmv_bytes(csr, value_bytes):
    """Algorithmic bytes of one SpMV: row_ptr + col_ind + val + x read + y write."""
    return (csr.m + 1) * 4 + csr.nnz * (4 + value_bytes) + csr.n * value_bytes + csr.m * value_bytes


def spmm_bytes(csr, n_cols, value_bytes):
    """Algorithmic bytes of one SpMM: A + B read + C write."""
    return (csr.m + 1) * 4 + csr.nnz * (4 + value_bytes) + (csr.n + csr.m) * n_cols * value_bytes
