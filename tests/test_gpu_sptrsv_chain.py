"""Triangular solves whose levels hold one row each (banded factors, bidiagonal and tridiagonal
triangles): a single wavefront walks such a run with the newest solution in a register, adds in
the serial loop's order (cpp/sparse_csr_cpu.cpp:672-718) and divides by a three-operation
shortcut that it checks against a true division.  Everything here is compared bit for bit,
signed zeros included, with the serial oracle.
"""
import numpy as np
import pytest
import scipy.sparse as sps

import oracle
from numml_amd import numml_torch_cpp as ext
from util import assert_close, host, randn, to_dev

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]


def assert_bits(a, ref, what):
    a, ref = np.asarray(a), np.asarray(ref)
    assert a.shape == ref.shape and a.dtype == ref.dtype, f"{what}: {a.shape}/{a.dtype} vs {ref.shape}/{ref.dtype}"
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(a), nan), f"{what}: NaNs in other places"
    same = (a == ref) & (np.signbit(a) == np.signbit(ref))
    bad = ~(same | nan)
    assert not bad.any(), f"{what}: {int(bad.sum())} of {a.size} entries differ, first at {int(np.argmax(bad))}"


def csr(M, dtype):
    M = sps.csr_matrix(M).astype(dtype)
    M.sort_indices()
    return M.data.copy(), M.indices.astype(np.int64), M.indptr.astype(np.int64), M.shape[0]


def banded_lower(n, width, seed, dtype, keep=1.0):
    """Lower triangle with `width` sub-diagonals (each entry kept with probability `keep`, the first
    sub-diagonal always), small off-diagonal values and a diagonal near 1.25."""
    rng = np.random.default_rng(seed)
    rows, cols, vals = [], [], []
    for k in range(1, width + 1):
        m = n - k
        if m <= 0:
            break
        on = np.ones(m, bool) if k == 1 else rng.random(m) < keep
        r = np.arange(k, n)[on]
        rows.append(r)
        cols.append(r - k)
        vals.append(rng.uniform(-1, 1, r.size) * (0.9 / width))
    rows.append(np.arange(n)); cols.append(np.arange(n)); vals.append(rng.uniform(1.0, 1.5, n) * rng.choice([-1, 1], n))
    return sps.csr_matrix((np.concatenate(vals), (np.concatenate(rows), np.concatenate(cols))), shape=(n, n))


def solve_and_compare(dev, M, lower, unit, dtype, what, b=None, expect_chain=None, exact=True):
    d, i, p, n = csr(M, dtype)
    b = randn(11, n, dtype) if b is None else b.astype(dtype)
    g = randn(12, n, dtype)
    x_ref = oracle.sptrsv_forward(n, n, d, i, p, lower, unit, b)
    gA_ref, gb_ref = oracle.sptrsv_backward(g, x_ref, n, n, d, i, p, lower, unit)
    D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
    chain = ext.sptrsv_chain_levels(n, I, P, lower)
    if expect_chain is not None:
        levels = ext.sptrsv_schedule(n, I, P, lower)[0]
        for dirn in (0, 1):
            if expect_chain:
                assert chain[dirn] >= levels - 70, f"{what}: {chain[dirn]} of {levels} levels on the chain kernels"
            else:
                assert chain[dirn] == 0, f"{what}: no chain expected, got {chain}"
    same = assert_bits if exact else assert_close
    x = ext.sptrsv_forward(n, n, D, I, P, lower, unit, Bv)
    same(host(x), x_ref, f"{what} x")
    gA, gb = ext.sptrsv_backward(Gv, x, n, n, D, I, P, lower, unit, Bv)
    if not exact:       # the oracle's gradients start from its own x
        gA_ref, gb_ref = oracle.sptrsv_backward(g, host(x), n, n, d, i, p, lower, unit)
    same(host(gb), gb_ref, f"{what} grad_b")
    same(host(gA), gA_ref, f"{what} grad_A")
    return chain


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lower", [True, False])
@pytest.mark.parametrize("unit", [False, True])
def test_bidiagonal_and_banded_chains(dev, dtype, lower, unit):
    side = (lambda M: M) if lower else (lambda M: M.T)
    # 5000 levels of one row: two launches (4096 levels each at most), the second starts from the first's last row
    solve_and_compare(dev, side(banded_lower(5000, 1, 1, dtype)), lower, unit, dtype, "bidiagonal 5000", expect_chain=True)
    # every row waits for all of the 64 rows before it (the pattern of a banded factor)
    solve_and_compare(dev, side(banded_lower(700, 64, 2, dtype)), lower, unit, dtype, "band 64 full", expect_chain=True)
    # ragged band, a length that is no multiple of 64, more than one block
    solve_and_compare(dev, side(banded_lower(333, 50, 3, dtype, keep=0.8)), lower, unit, dtype, "band 50 ragged",
                      expect_chain=True)
    # a band that reaches further back than 64 rows stays with the workgroup kernels (64 lanes share
    # a row there and add their parts across the group: equal to rounding)
    solve_and_compare(dev, side(banded_lower(400, 70, 4, dtype)), lower, unit, dtype, "band 70", expect_chain=False,
                      exact=False)
    # a narrow band streams 64-wide coefficient rows like a wide one
    solve_and_compare(dev, side(banded_lower(300, 3, 5, dtype)), lower, unit, dtype, "band 3", expect_chain=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lower", [True, False])
def test_chain_behind_a_block_of_independent_rows(dev, dtype, lower):
    # 600 rows that wait for nothing, then 500 rows that each wait for the row before them and for
    # rows of the first block: those come first in the accumulation order and are summed ahead
    rng = np.random.default_rng(7)
    n0, n1 = 600, 500
    n = n0 + n1
    for width, name in ((1, "narrow"), (40, "wide")):
        L = sps.lil_matrix((n, n))
        L.setdiag(rng.uniform(1.0, 1.5, n))
        for r in range(n0, n):
            for c in rng.choice(n0, 3, replace=False):
                L[r, c] = rng.uniform(-0.2, 0.2)
            for k in range(1, width + 1):
                if r - k >= n0 and (k == 1 or rng.random() < 0.7):
                    L[r, r - k] = rng.uniform(-1, 1) * 0.5 / width
        M = L.tocsr() if lower else L.tocsr().T
        # (without a chain, rows of 40 entries share lanes and match the serial sum to rounding)
        chain = solve_and_compare(dev, M, lower, False, dtype, f"block + {name} chain", exact=lower or width == 1)
        # (in the levels of the upper triangle L^T the rows of the block share levels with the
        # chain's rows, so there is no run of one-row levels to take)
        if lower:
            assert chain[0] >= n1 - 70, chain
    # an order the chain kernels must refuse: chain rows on the even indices, and between a row's two
    # chain neighbours a dependency on an odd row that belongs to no chain
    m = 400
    L = sps.lil_matrix((2 * m, 2 * m))
    L.setdiag(rng.uniform(1.0, 1.5, 2 * m))
    for k in range(2, m):
        L[2 * k, 2 * k - 4] = 0.1
        L[2 * k, 2 * k - 3] = 0.2          # outside the chain, between the two chain entries
        L[2 * k, 2 * k - 2] = -0.3
    L[2, 0] = 0.25
    M = L.tocsr() if lower else L.tocsr().T
    chain = solve_and_compare(dev, M, lower, False, dtype, "interleaved order")
    if lower:
        assert chain[0] == 0, chain


@pytest.mark.parametrize("dtype", DTYPES)
def test_values_the_division_shortcut_does_not_cover(dev, dtype):
    # zeros of either sign in the right-hand side, a zero and a missing diagonal, infinities and NaN:
    # the block that meets them is solved again with true divisions, and the launch goes on that way
    n = 900
    for width in (1, 30):
        M = banded_lower(n, width, 21 + width, dtype).tolil()
        b = randn(5, n, np.float64)
        b[100:140] = 0.0
        b[200:230] = -0.0
        solve_and_compare(dev, M, True, False, dtype, f"signed zeros, band {width}", b=b)
        solve_and_compare(dev, M, True, True, dtype, f"signed zeros, unit, band {width}", b=b)
        Mz = M.copy()
        Mz[450, 450] = 0.0                      # no diagonal entry in row 450: a division by zero
        solve_and_compare(dev, sps.csr_matrix(Mz), True, False, dtype, f"missing diagonal, band {width}", b=b)
        b2 = randn(6, n, np.float64)
        b2[300] = np.inf
        solve_and_compare(dev, M, True, False, dtype, f"infinite right-hand side, band {width}", b=b2)
        b2[300] = np.nan
        solve_and_compare(dev, M, True, False, dtype, f"NaN right-hand side, band {width}", b=b2)
        # huge and tiny magnitudes: quotients that overflow, underflow or are subnormal
        big = np.finfo(dtype).max / 4
        b3 = randn(8, n, np.float64)
        b3[::7] *= big
        b3[3::7] *= float(np.finfo(dtype).tiny)
        solve_and_compare(dev, M, True, False, dtype, f"extreme magnitudes, band {width}", b=b3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lower", [True, False])
def test_a_dense_row_and_a_dense_column(dev, dtype, lower):
    # arrowhead triangles of 5000 rows: one row (and, in the other triangle, one column) of 5000
    # entries, which the level analysis packs by a wavefront instead of a lane (the order of a row's
    # dependencies is the one of the serial walk, cpp/sparse_csr_cpu.cpp:672-718; rows this long are
    # added across lanes, hence the tolerance)
    n = 5000
    rng = np.random.default_rng(31)
    for dense_row in (True, False):
        L = sps.lil_matrix((n, n))
        L.setdiag(rng.uniform(2.0, 3.0, n))
        if dense_row:
            L[n - 1, :n - 1] = rng.uniform(-1, 1, n - 1) / n
        else:
            L[1:, 0] = (rng.uniform(-1, 1, n - 1) / n).reshape(-1, 1)
        for k in range(5, n, 7):
            L[k, k - 3] = 0.1
        M = L.tocsr() if lower else L.tocsr().T
        solve_and_compare(dev, M, lower, False, dtype, f"arrowhead, dense {'row' if dense_row else 'column'}", exact=False)
        solve_and_compare(dev, M, lower, True, dtype, f"unit arrowhead, dense {'row' if dense_row else 'column'}",
                          exact=False)
