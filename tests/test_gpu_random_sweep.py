"""Randomised shapes against the serial oracle: many small matrices whose sizes, densities and
row lengths are drawn per seed, so that the tile edges of the kernels (rows that end at a chunk
boundary, empty rows at either end, rows just over the long-row limits, dense widths that are
not a multiple of a wavefront, triangles whose rows are long or short) are hit by construction
rather than by luck of a hand-picked case.  Every case prints its name first.
"""
import os

import numpy as np
import pytest
import scipy.sparse as sps

import numml_amd
import oracle
from numml_amd import generators as G
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

SEEDS = list(range(int(os.environ.get("NM_SWEEP_SEEDS", "24"))))   # more seeds for a longer soak


def _draw(seed, dtype, square=False):
    rng = np.random.default_rng(1000 + seed)
    kind = seed % 4
    rows = int(rng.integers(1, 700))
    cols = rows if square else int(rng.integers(1, 900))
    if kind == 0:       # uniform density, some rows empty
        m = G.random_csr(rows, cols, float(rng.uniform(0.002, 0.2)), seed, dtype)
    elif kind == 1:     # ragged: lengths uniform in [0, max_len]
        m = G.ragged_csr(rows, cols, int(rng.integers(1, min(cols, 80) + 1)), seed, dtype)
    elif kind == 2:     # a few very long rows among short ones
        m = G.powerlaw(rows, cols, target_nnz=int(rows * rng.uniform(2, 12)), max_deg=cols, seed=seed, dtype=dtype)
    else:               # long rows only: lengths around the limits of the row-splitting paths
        cols = max(cols, 600) if not square else cols
        m = G.ragged_csr(rows if rows < 60 else 60, cols, min(cols, int(rng.integers(500, 1100))), seed, dtype,
                         min_len=min(cols, 480))
        if square:
            d, i, p, (r, c) = m
            n = max(r, c)
            m = (d, i, np.concatenate([p, np.full(n - r, p[-1])]).astype(np.int64), (n, n))
    return m


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("seed", SEEDS)
def test_products(dev, seed, dtype):
    ext = numml_amd.load_compiled()
    d, i, p, (rows, cols) = _draw(seed, dtype)
    print(f"case seed={seed} {dtype.__name__} {rows}x{cols} nnz={d.shape[0]}", flush=True)
    D, I, P = to_dev(dev, d, i, p)
    # SpMV
    x, g = randn(seed, cols, dtype), randn(seed + 1, rows, dtype)
    X, Gv = to_dev(dev, x, g)
    assert_close(host(ext.spgemv_forward(rows, cols, D, I, P, X)), oracle.spgemv_forward(rows, cols, d, i, p, x), "y")
    gA, gx = ext.spgemv_backward(Gv, rows, cols, D, I, P, X)
    gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
    assert_same(host(gA), gA_ref, "spmv grad_A")
    assert_close(host(gx), gx_ref, "spmv grad_x")
    # SpMM at widths around the wavefront size
    for n in (1, 7, 16, 20, 32, 64, 65, 130)[seed % 2::2]:
        B, gC = randn(seed + 2, (cols, n), dtype), randn(seed + 3, (rows, n), dtype)
        Bd, gCd = to_dev(dev, B, gC)
        assert_close(host(ext.spdmm_forward(rows, cols, D, I, P, Bd)), oracle.spdmm_forward(rows, cols, d, i, p, B),
                     f"C n={n}")
        gA, gB = ext.spdmm_backward(rows, cols, D, I, P, Bd, gCd)
        gA_ref, gB_ref = oracle.spdmm_backward(rows, cols, d, i, p, B, gC)
        assert_close(host(gA), gA_ref, f"spmm grad_A n={n}")
        assert_close(host(gB), gB_ref, f"spmm grad_B n={n}")
    # transpose, row sums, diagonal, dense copy
    out = ext.csr_transpose_forward(rows, cols, D, I, P)
    for got, want, what in zip(out, oracle.csr_transpose(rows, cols, d, i, p), ("At_data", "At_indices", "At_indptr", "map")):
        assert_same(host(got), want, what)
    assert_close(host(ext.csr_row_sum_forward(rows, cols, D, I, P)), oracle.csr_row_sum_forward(rows, cols, d, i, p), "row sums")
    assert_same(host(ext.csr_extract_diagonal_forward(rows, cols, D, I, P)),
                oracle.csr_extract_diagonal_forward(rows, cols, d, i, p), "diagonal")
    if rows * cols <= 200_000:
        assert_same(host(ext.csr_to_dense_forward(rows, cols, D, I, P)), oracle.csr_to_dense_forward(rows, cols, d, i, p), "dense")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("seed", SEEDS)
def test_sparse_sparse(dev, seed, dtype):
    ext = numml_amd.load_compiled()
    d, i, p, (rows, cols) = _draw(seed, dtype)
    if seed % 4 == 3:      # the long-row draw squared would be dense: keep its pattern but thin the partner
        d2, i2, p2, (r2, c2) = G.random_csr(cols, 300, 0.01, seed, dtype)
    else:
        d2, i2, p2, (r2, c2) = G.random_csr(cols, int(np.random.default_rng(seed).integers(1, 500)), 0.03, seed + 50, dtype)
    print(f"case seed={seed} {dtype.__name__} ({rows}x{cols}) @ ({r2}x{c2})", flush=True)
    A, B = to_dev(dev, d, i, p), to_dev(dev, d2, i2, p2)
    C = ext.spgemm_forward(rows, cols, *A, r2, c2, *B)
    C_ref = oracle.spgemm_forward(rows, cols, d, i, p, r2, c2, d2, i2, p2)
    assert_same(host(C[2]), C_ref[2], "C_indptr")
    assert_same(host(C[1]), C_ref[1], "C_indices")
    assert_close(host(C[0]), C_ref[0], "C_data")
    gC = randn(seed + 4, C_ref[0].shape[0], dtype)
    gA, gB = ext.spgemm_backward(to_dev(dev, gC)[0], C[1], C[2], rows, cols, *A, r2, c2, *B)
    gA_ref, gB_ref = oracle.spgemm_backward(gC, C_ref[1], C_ref[2], rows, cols, d, i, p, r2, c2, d2, i2, p2)
    assert_close(host(gA), gA_ref, "spgemm grad_A")
    assert_close(host(gB), gB_ref, "spgemm grad_B")
    # A + beta * A' on a second pattern of the same shape
    e, j, q, _ = G.random_csr(rows, cols, 0.05, seed + 99, dtype)
    import torch
    al, be = torch.tensor(1.5), torch.tensor(-0.25)
    S = ext.splincomb_forward(rows, cols, al, *A, be, *to_dev(dev, e, j, q))
    S_ref = oracle.splincomb_forward(rows, cols, 1.5, d, i, p, -0.25, e, j, q)
    for got, want, what in zip(S, S_ref, ("S_data", "S_indices", "S_indptr")):
        assert_same(host(got), want, what)
    gS = randn(seed + 5, S_ref[0].shape[0], dtype)
    gs = ext.splincomb_backward(rows, cols, al, *A, be, *to_dev(dev, e, j, q), to_dev(dev, gS)[0], S[1], S[2])
    for got, want, what in zip(gs, oracle.splincomb_backward(rows, cols, 1.5, d, i, p, -0.25, e, j, q, gS, S_ref[1], S_ref[2]),
                               ("grad_A", "grad_B")):
        assert_same(host(got), want, f"lincomb {what}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("seed", SEEDS)
def test_triangular_and_direct_solves(dev, seed, dtype):
    ext = numml_amd.load_compiled()
    rng = np.random.default_rng(2000 + seed)
    n = int(rng.integers(1, 1500))
    # rows from a couple of dependencies (fixed-width kernels) to dozens (lanes-per-row kernel)
    density = [2.0 / n, 6.0 / n, 0.02, 0.15][seed % 4]
    for lower in (True, False):
        for unit in (False, True):
            d, i, p, _ = G.random_tri(n, min(density, 1.0), seed, lower=lower, dtype=dtype)
            print(f"case seed={seed} {dtype.__name__} n={n} nnz={d.shape[0]} lower={lower} unit={unit}", flush=True)
            b, g = randn(seed, n, dtype), randn(seed + 1, n, dtype)
            x_ref = oracle.sptrsv_forward(n, n, d, i, p, lower, unit, b)
            D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
            x = ext.sptrsv_forward(n, n, D, I, P, lower, unit, Bv)
            assert_close(host(x), x_ref, "x")
            gA, gb = ext.sptrsv_backward(Gv, x, n, n, D, I, P, lower, unit, Bv)
            gA_ref, gb_ref = oracle.sptrsv_backward(g, host(x), n, n, d, i, p, lower, unit)
            assert_close(host(gb), gb_ref, "grad_b")
            assert_close(host(gA), gA_ref, "grad_A")
    # LU of a diagonally dominant matrix on a random pattern
    m = min(n, 400)
    a = sps.random(m, m, min(4.0 / m, 1.0), random_state=seed, dtype=np.float64)
    a = (a + sps.eye(m) * (abs(a).sum(1).max() + 1.0)).tocsr()
    a.sort_indices()
    d, i, p = a.data.astype(dtype), a.indices.astype(np.int64), a.indptr.astype(np.int64)
    print(f"case seed={seed} {dtype.__name__} splu n={m} nnz={d.shape[0]}", flush=True)
    out = ext.splu(m, m, *to_dev(dev, d, i, p))
    for got, want, what in zip(out, oracle.splu(m, m, d, i, p), ("M_data", "M_indices", "M_indptr", "Mt_data", "Mt_indices", "Mt_indptr")):
        assert_same(host(got), want, what)


# ---- the same comparisons over grids of thousands of workgroups ----------------------
# Wavefronts of a workgroup that share LDS without a barrier, and workgroups that meet in
# global memory, only get out of step on inputs of this size.

def _big(seed, dtype, rows, cols, lens):
    """CSR with the given row lengths, distinct sorted uniform columns, N(0,1) values."""
    rng = np.random.default_rng(5000 + seed)
    lens = np.minimum(lens, cols).astype(np.int64)
    indptr = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(lens, out=indptr[1:])
    row_of = np.repeat(np.arange(rows, dtype=np.int64), lens)
    key = row_of * cols + rng.integers(0, cols, row_of.shape[0], dtype=np.int64)
    key.sort()
    while True:
        dup = np.flatnonzero(key[1:] == key[:-1]) + 1
        if dup.size == 0:
            break
        key[dup] = row_of[dup] * cols + rng.integers(0, cols, dup.size, dtype=np.int64)
        key.sort()
    return rng.standard_normal(key.shape[0]).astype(dtype), key - row_of * cols, indptr, (rows, cols)


def _big_draw(seed, dtype):
    rng = np.random.default_rng(4000 + seed)
    rows, cols = int(rng.integers(60_000, 220_000)), int(rng.integers(40_000, 200_000))
    kind = seed % 3
    if kind == 0:      # 0-12 entries per row, many empty rows
        lens = rng.integers(0, 13, rows) * (rng.random(rows) < 0.8)
    elif kind == 1:    # 15-40 entries per row: blocks of rows that do not fit the LDS tiles
        lens = rng.integers(15, 41, rows)
    else:              # short rows with a heavy tail up to thousands of entries
        lens = np.clip(rng.zipf(1.9, rows), 1, 6000)
    return _big(seed, dtype, rows, cols, lens)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("seed", range(int(os.environ.get("NM_SWEEP_BIG_FIRST", "0")),
                                         int(os.environ.get("NM_SWEEP_BIG_FIRST", "0")) + int(os.environ.get("NM_SWEEP_BIG", "6"))))
def test_many_workgroups(dev, seed, dtype):
    import torch
    ext = numml_amd.load_compiled()
    d, i, p, (rows, cols) = _big_draw(seed, dtype)
    print(f"case seed={seed} {dtype.__name__} {rows}x{cols} nnz={d.shape[0]} longest row {np.diff(p).max()}", flush=True)
    D, I, P = to_dev(dev, d, i, p)
    x, g = randn(seed, cols, dtype), randn(seed + 1, rows, dtype)
    X, Gv = to_dev(dev, x, g)
    assert_close(host(ext.spgemv_forward(rows, cols, D, I, P, X)), oracle.spgemv_forward(rows, cols, d, i, p, x), "y")
    gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
    for mode in ("eager", "atomic"):
        ext.set_backward_mode(mode)
        try:
            gA, gx = ext.spgemv_backward(Gv, rows, cols, D, I, P, X)
        finally:
            ext.set_backward_mode("eager")
        assert_same(host(gA), gA_ref, f"spmv grad_A ({mode})")
        assert_close(host(gx), gx_ref, f"spmv grad_x ({mode})")
    n = (4, 16, 33, 64, 7, 100)[seed % 6]
    B, gC = randn(seed + 2, (cols, n), dtype), randn(seed + 3, (rows, n), dtype)
    Bd, gCd = to_dev(dev, B, gC)
    assert_close(host(ext.spdmm_forward(rows, cols, D, I, P, Bd)), oracle.spdmm_forward(rows, cols, d, i, p, B), f"C n={n}")
    gA, gB = ext.spdmm_backward(rows, cols, D, I, P, Bd, gCd)
    gA_ref, gB_ref = oracle.spdmm_backward(rows, cols, d, i, p, B, gC)
    assert_close(host(gA), gA_ref, f"spmm grad_A n={n}")
    assert_close(host(gB), gB_ref, f"spmm grad_B n={n}")
    out = ext.csr_transpose_forward(rows, cols, D, I, P)
    for got, want, what in zip(out, oracle.csr_transpose(rows, cols, d, i, p), ("At_data", "At_indices", "At_indptr", "map")):
        assert_same(host(got), want, what)
    assert_close(host(ext.csr_row_sum_forward(rows, cols, D, I, P)), oracle.csr_row_sum_forward(rows, cols, d, i, p), "row sums")
    assert_same(host(ext.csr_extract_diagonal_forward(rows, cols, D, I, P)),
                oracle.csr_extract_diagonal_forward(rows, cols, d, i, p), "diagonal")
    # linear combination with a second pattern of the same shape
    e, j, q, _ = _big(seed + 100, dtype, rows, cols, np.random.default_rng(seed).integers(0, 9, rows))
    al, be = torch.tensor(1.5), torch.tensor(-0.25)
    E = to_dev(dev, e, j, q)
    S = ext.splincomb_forward(rows, cols, al, D, I, P, be, *E)
    S_ref = oracle.splincomb_forward(rows, cols, 1.5, d, i, p, -0.25, e, j, q)
    for got, want, what in zip(S, S_ref, ("S_data", "S_indices", "S_indptr")):
        assert_same(host(got), want, what)
    gS = randn(seed + 5, S_ref[0].shape[0], dtype)
    gs = ext.splincomb_backward(rows, cols, al, D, I, P, be, *E, to_dev(dev, gS)[0], S[1], S[2])
    for got, want, what in zip(gs, oracle.splincomb_backward(rows, cols, 1.5, d, i, p, -0.25, e, j, q, gS, S_ref[1], S_ref[2]),
                               ("grad_A", "grad_B")):
        assert_same(host(got), want, f"lincomb {what}")
    # product with a thin second operand
    m = int(np.random.default_rng(seed).integers(2_000, 50_000))
    d2, i2, p2, _ = _big(seed + 200, dtype, cols, m, np.random.default_rng(seed + 1).integers(0, 7, cols))
    B2 = to_dev(dev, d2, i2, p2)
    C = ext.spgemm_forward(rows, cols, D, I, P, cols, m, *B2)
    C_ref = oracle.spgemm_forward(rows, cols, d, i, p, cols, m, d2, i2, p2)
    assert_same(host(C[2]), C_ref[2], "C_indptr")
    assert_same(host(C[1]), C_ref[1], "C_indices")
    assert_close(host(C[0]), C_ref[0], "C_data")
    gCs = randn(seed + 4, C_ref[0].shape[0], dtype)
    gA, gB = ext.spgemm_backward(to_dev(dev, gCs)[0], C[1], C[2], rows, cols, D, I, P, cols, m, *B2)
    gA_ref, gB_ref = oracle.spgemm_backward(gCs, C_ref[1], C_ref[2], rows, cols, d, i, p, cols, m, d2, i2, p2)
    assert_close(host(gA), gA_ref, "spgemm grad_A")
    assert_close(host(gB), gB_ref, "spgemm grad_B")


def _big_triangle(seed, dtype, n, deps, window, lower):
    """Triangular CSR: row i holds `deps` entries (fewer near the corner) among the `window` rows
    before it (after it for an upper triangle), N(0, 0.1) values, and a diagonal in [2, 3)."""
    rng = np.random.default_rng(7000 + seed)
    lens = np.minimum(np.arange(n), deps).astype(np.int64)
    row_of = np.repeat(np.arange(n, dtype=np.int64), lens)
    reach = np.minimum(row_of, window)
    off = 1 + (rng.random(row_of.shape[0]) * reach).astype(np.int64)
    key = np.unique(row_of * (window + 1) + np.minimum(off, reach))          # duplicates dropped
    r, c = key // (window + 1), key // (window + 1) - key % (window + 1)
    r, c = np.concatenate([r, np.arange(n)]), np.concatenate([c, np.arange(n)])
    v = np.concatenate([rng.standard_normal(key.shape[0]) * 0.1, 2.0 + rng.random(n)])
    M = sps.csr_matrix((v, (r, c)), shape=(n, n))
    if not lower:
        M = M.T.tocsr()
    M.sort_indices()
    return M.data.astype(dtype), M.indices.astype(np.int64), M.indptr.astype(np.int64)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("lower", [True, False])
@pytest.mark.parametrize("deps,window", [(3, 400), (6, 3000), (14, 1500)])
def test_triangular_solves_over_thousands_of_levels(dev, dtype, lower, deps, window):
    ext = numml_amd.load_compiled()
    n = 150_000
    d, i, p = _big_triangle(deps, dtype, n, deps, window, lower)
    print(f"case {dtype.__name__} n={n} nnz={d.shape[0]} lower={lower} deps={deps} window={window}", flush=True)
    b, g = randn(deps, n, dtype), randn(deps + 1, n, dtype)
    D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
    for unit in (False, True):
        x_ref = oracle.sptrsv_forward(n, n, d, i, p, lower, unit, b)
        x = ext.sptrsv_forward(n, n, D, I, P, lower, unit, Bv)
        assert_close(host(x), x_ref, f"x unit={unit}")
        gA, gb = ext.sptrsv_backward(Gv, x, n, n, D, I, P, lower, unit, Bv)
        gA_ref, gb_ref = oracle.sptrsv_backward(g, host(x), n, n, d, i, p, lower, unit)
        assert_close(host(gb), gb_ref, f"grad_b unit={unit}")
        assert_close(host(gA), gA_ref, f"grad_A unit={unit}")
