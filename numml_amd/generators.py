"""Seeded synthetic CSR matrices for the benchmark and the parity tests.

Every generator returns ``(data, indices, indptr, shape)`` as NumPy arrays with
int64 structure and ascending column indices inside each row, which is the
layout the reference's kernels assume (cpp/sparse_csr_cpu.cpp:24-25 reads the
structure through int64 accessors; the merge in :261-274 and the ``break`` in
:680-681 need sorted rows).  Random numbers come from
``numpy.random.default_rng(seed)`` only, so the same call gives the same matrix
on every machine.
"""
import numpy as np

__all__ = [
    "poisson2d", "laplace3d", "poisson2d_lower", "powerlaw", "tridiag", "bidiag",
    "random_csr", "random_tri",
]


def _stencil_csr(offsets_valid, n_rows):
    """Assemble a stencil matrix from per-offset (offset, valid-mask, value) triples.

    ``offsets_valid`` lists the stencil legs in ascending column-offset order, so
    the entries of each row come out sorted without a sort.
    """
    counts = np.zeros(n_rows, dtype=np.int64)
    for _, valid, _ in offsets_valid:
        counts += valid
    indptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(counts, out=indptr[1:])
    nnz = int(indptr[-1])
    indices = np.empty(nnz, dtype=np.int64)
    data = np.empty(nnz, dtype=np.float64)
    cursor = indptr[:-1].copy()
    rows = np.arange(n_rows, dtype=np.int64)
    for off, valid, val in offsets_valid:
        pos = cursor[valid]
        indices[pos] = rows[valid] + off
        data[pos] = val
        cursor += valid
    return data, indices, indptr


def poisson2d(n, dtype=np.float64, jitter_seed=None):
    """5-point Laplacian on an n x n grid: 4 on the diagonal, -1 off it.

    With ``jitter_seed`` every stored value is multiplied by
    ``1 + 0.01 * U(-1, 1)`` drawn in storage order from that seed.
    """
    N = n * n
    r = np.arange(N, dtype=np.int64)
    a, b = r // n, r % n
    legs = [(-n, a > 0, -1.0), (-1, b > 0, -1.0), (0, np.ones(N, bool), 4.0),
            (1, b < n - 1, -1.0), (n, a < n - 1, -1.0)]
    data, indices, indptr = _stencil_csr(legs, N)
    if jitter_seed is not None:
        rng = np.random.default_rng(jitter_seed)
        data *= 1.0 + 0.01 * rng.uniform(-1.0, 1.0, data.shape[0])
    return data.astype(dtype), indices, indptr, (N, N)


def laplace3d(n, dtype=np.float64, jitter_seed=None):
    """7-point Laplacian on an n^3 grid: 6 on the diagonal, -1 off it.

    With ``jitter_seed`` only the off-diagonal values are scaled by
    ``1 + 0.01 * U(-1, 1)``; one draw is consumed per stored entry (diagonal
    draws are discarded) so the stream position is a function of nnz alone.
    """
    N = n * n * n
    r = np.arange(N, dtype=np.int64)
    a, b, c = r // (n * n), (r // n) % n, r % n
    legs = [(-n * n, a > 0, -1.0), (-n, b > 0, -1.0), (-1, c > 0, -1.0),
            (0, np.ones(N, bool), 6.0),
            (1, c < n - 1, -1.0), (n, b < n - 1, -1.0), (n * n, a < n - 1, -1.0)]
    data, indices, indptr = _stencil_csr(legs, N)
    if jitter_seed is not None:
        rng = np.random.default_rng(jitter_seed)
        u = rng.uniform(-1.0, 1.0, data.shape[0])
        offdiag = data < 0
        data[offdiag] *= 1.0 + 0.01 * u[offdiag]
    return data.astype(dtype), indices, indptr, (N, N)


def poisson2d_lower(n, dtype=np.float64, diag_seed=0):
    """Lower triangle (with diagonal) of :func:`poisson2d`; diagonal = 4 + U(0,1)."""
    N = n * n
    r = np.arange(N, dtype=np.int64)
    a, b = r // n, r % n
    legs = [(-n, a > 0, -1.0), (-1, b > 0, -1.0), (0, np.ones(N, bool), 4.0)]
    data, indices, indptr = _stencil_csr(legs, N)
    rng = np.random.default_rng(diag_seed)
    data[indptr[1:] - 1] = 4.0 + rng.uniform(0.0, 1.0, N)
    return data.astype(dtype), indices, indptr, (N, N)


def tridiag(n, dtype=np.float64, lo=-1.0, di=2.0, up=-1.0):
    """1-D Poisson matrix ``2I - E_-1 - E_+1`` (the reference tests' canonical case,
    numml/tests/test_spmv.py:9-10)."""
    r = np.arange(n, dtype=np.int64)
    legs = [(-1, r > 0, lo), (0, np.ones(n, bool), di), (1, r < n - 1, up)]
    data, indices, indptr = _stencil_csr(legs, n)
    return data.astype(dtype), indices, indptr, (n, n)


def bidiag(n, dtype=np.float64, lower=True, di=2.0, off=-1.0):
    """Bidiagonal ``2I - E_-1`` (or its transpose), the reference's triangular-solve
    timing matrix (demos/timing.py:520-558): n dependency levels of one row each."""
    r = np.arange(n, dtype=np.int64)
    if lower:
        legs = [(-1, r > 0, off), (0, np.ones(n, bool), di)]
    else:
        legs = [(0, np.ones(n, bool), di), (1, r < n - 1, off)]
    data, indices, indptr = _stencil_csr(legs, n)
    return data.astype(dtype), indices, indptr, (n, n)


def powerlaw(rows, cols, target_nnz=None, a=2.1, max_deg=10_000, seed=0,
             dtype=np.float32):
    """Random CSR with Zipf(a) row degrees clipped to [1, max_deg].

    Columns are uniform without replacement inside each row (sorted), values are
    U(0,1) normalised so every row sums to 1.  A raw Zipf(2.1) draw has mean
    degree ~4.4; with ``target_nnz`` the degrees are scaled by
    ``target_nnz / sum(deg)`` before clipping so the matrix keeps the power-law
    tail and lands near the requested size.
    """
    rng = np.random.default_rng(seed)
    deg = np.clip(rng.zipf(a, rows), 1, max_deg).astype(np.int64)
    if target_nnz is not None:
        s = target_nnz / float(deg.sum())
        deg = np.clip(np.ceil(s * deg), 1, max_deg).astype(np.int64)
    deg = np.minimum(deg, cols)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(deg, out=indptr[1:])
    nnz = int(indptr[-1])
    row_of = np.repeat(np.arange(rows, dtype=np.int64), deg)
    key = row_of * cols + rng.integers(0, cols, nnz, dtype=np.int64)
    key.sort()
    # redraw duplicate (row, col) pairs until every row holds distinct columns
    while True:
        dup = np.flatnonzero(key[1:] == key[:-1]) + 1
        if dup.size == 0:
            break
        key[dup] = row_of[dup] * cols + rng.integers(0, cols, dup.size, dtype=np.int64)
        key.sort()
    indices = key - row_of * cols
    data = rng.uniform(0.0, 1.0, nnz)
    rowsum = np.add.reduceat(data, indptr[:-1])
    data /= np.repeat(rowsum, deg)
    return data.astype(dtype), indices, indptr, (rows, cols)


def random_csr(rows, cols, density, seed, dtype=np.float64, empty_rows=True):
    """Uniformly random pattern with N(0,1) values; some rows are left empty on purpose."""
    rng = np.random.default_rng(seed)
    mask = rng.random((rows, cols)) < density
    if empty_rows and rows > 3:
        mask[rng.integers(0, rows, max(1, rows // 8))] = False
    r, c = np.nonzero(mask)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(np.bincount(r, minlength=rows), out=indptr[1:])
    data = rng.standard_normal(r.shape[0]).astype(dtype)
    return data, c.astype(np.int64), indptr, (rows, cols)


def random_tri(n, density, seed, lower=True, dtype=np.float64, diag=True,
               wrong_side=0.0):
    """Random triangular matrix: N(0,1) off the diagonal, 2 + U(0,1) on it.

    ``wrong_side`` > 0 also stores a few entries on the other side of the
    diagonal; the solve ignores them but its backward still gives them a
    gradient (cpp/sparse_csr_cpu.cpp:750-755).
    """
    rng = np.random.default_rng(seed)
    m = rng.random((n, n)) < density
    m = np.tril(m, -1) if lower else np.triu(m, 1)
    if wrong_side > 0:
        w = rng.random((n, n)) < wrong_side
        m |= np.triu(w, 1) if lower else np.tril(w, -1)
    if diag:
        m |= np.eye(n, dtype=bool)
    r, c = np.nonzero(m)
    vals = rng.standard_normal(r.shape[0]) * 0.5
    vals[r == c] = 2.0 + rng.uniform(0, 1, int((r == c).sum()))
    indptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(r, minlength=n), out=indptr[1:])
    return vals.astype(dtype), c.astype(np.int64), indptr, (n, n)


def ragged_csr(rows, cols, max_len, seed, dtype=np.float64, min_len=0):
    """Rows of independently drawn lengths in [min_len, max_len] (uniform), columns drawn
    without replacement and sorted, N(0,1) values: mixes empty, short and longer rows."""
    rng = np.random.default_rng(seed)
    lens = rng.integers(min_len, min(max_len, cols) + 1, rows)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(lens, out=indptr[1:])
    indices = np.empty(indptr[-1], dtype=np.int64)
    for r in range(rows):
        indices[indptr[r]:indptr[r + 1]] = np.sort(rng.choice(cols, lens[r], replace=False))
    data = rng.standard_normal(indptr[-1]).astype(dtype)
    return data, indices, indptr, (rows, cols)
