"""Linear combination, dense copy, row sums and diagonal on a HIP device.

Compared with the CPU oracle (cpp/sparse_csr_cpu.cpp:387-560, 1050-1213), through
both bindings and through the ``SparseCSRTensor`` surface with gradients.
Structure and copied values are exact; the linear combination is two products
and one sum per entry in the value type, also exact; row sums are bitwise for
rows summed in storage order and within util.RTOL (1e-5 / 1e-12) for rows long
enough to be reduced by a wavefront.
"""
import numpy as np
import pytest
import torch

import numml_amd
import oracle
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as mirror
from numml_amd import sparse as sp
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]


@pytest.fixture(params=["compiled", "ctypes"])
def ext(request):
    return numml_amd.load_compiled() if request.param == "compiled" else mirror


def _pairs(dtype):
    yield "stencils", G.poisson2d(30, dtype, 1), G.poisson2d(30, dtype, 2)                   # same pattern
    yield "tri_vs_id", G.tridiag(500, dtype), (np.ones(500, dtype), np.arange(500), np.arange(501), (500, 500))
    yield "random", G.random_csr(300, 260, 0.05, 1, dtype), G.random_csr(300, 260, 0.08, 2, dtype)
    yield "disjointish", G.random_csr(64, 900, 0.01, 3, dtype), G.random_csr(64, 900, 0.3, 4, dtype)
    yield "powerlaw", (G.powerlaw(3000, 3000, 40000, max_deg=2500, seed=5, dtype=dtype),
                       G.powerlaw(3000, 3000, 30000, max_deg=2500, seed=6, dtype=dtype))[0], \
        G.powerlaw(3000, 3000, 30000, max_deg=2500, seed=6, dtype=dtype)
    # rows of ~40 entries: a tile of 256 rows does not fit LDS and is worked off in runs of rows
    yield "runs_of_rows", G.random_csr(700, 400, 0.1, 8, dtype), G.random_csr(700, 400, 0.12, 9, dtype)
    # rows too long for LDS in both operands, in one operand only, and next to short rows
    yield "long_both", G.random_csr(5, 20000, 0.3, 10, dtype, empty_rows=False), G.random_csr(5, 20000, 0.25, 11, dtype)
    yield "long_a_only", G.random_csr(3, 10000, 0.5, 12, dtype), G.random_csr(3, 10000, 0.001, 13, dtype)
    yield "long_b_only", G.random_csr(3, 10000, 0.001, 14, dtype), G.random_csr(3, 10000, 0.5, 15, dtype)
    yield "long_and_short", G.powerlaw(3000, 12000, 60000, max_deg=8000, seed=16, dtype=dtype), \
        G.powerlaw(3000, 12000, 50000, max_deg=8000, seed=17, dtype=dtype)
    yield "empty_a", (np.zeros(0, dtype), np.zeros(0, np.int64), np.zeros(8, np.int64), (7, 5)), \
        G.random_csr(7, 5, 0.4, 7, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_splincomb_forward_backward(dev, ext, dtype):
    for name, (ad, ai, ap, (r, c)), (bd, bi, bp, _) in _pairs(dtype):
        ai, ap, bi, bp = (np.asarray(v, np.int64) for v in (ai, ap, bi, bp))
        for alpha, beta in ((1.0, 1.0), (1.0, -1.0), (0.75, -2.5)):
            Cd_ref, Ci_ref, Cp_ref = oracle.splincomb_forward(r, c, alpha, ad, ai, ap, beta, bd, bi, bp)
            AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
            Cd, Ci, Cp = ext.splincomb_forward(r, c, torch.tensor(alpha), AD, AI, AP, torch.tensor(beta), BD, BI, BP)
            assert_same(host(Cp), Cp_ref, f"{name} C_indptr")
            assert_same(host(Ci), Ci_ref, f"{name} C_indices")
            assert_same(host(Cd), Cd_ref, f"{name} C_data")
            g = randn(3, Cd_ref.shape[0], dtype)
            gA, gB = ext.splincomb_backward(r, c, torch.tensor(alpha), AD, AI, AP, torch.tensor(beta), BD, BI, BP,
                                            to_dev(dev, g)[0], Ci, Cp)
            gA_ref, gB_ref = oracle.splincomb_backward(r, c, alpha, ad, ai, ap, beta, bd, bi, bp, g, Ci_ref, Cp_ref)
            assert_same(host(gA), gA_ref, f"{name} grad_A")
            assert_same(host(gB), gB_ref, f"{name} grad_B")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mode", ["planned", "eager"])
def test_splincomb_on_cached_maps(dev, dtype, mode):
    # The same two patterns with new values and new coefficients in every call, as in a loop over
    # A - B: the compiled binding records the maps of the combination (at the second sighting of the
    # pair, at the first in eager mode) and then fills C in one pass and gathers the gradients; every
    # call must give the bits of the serial merge (cpp/sparse_csr_cpu.cpp:387-560).
    ext = numml_amd.load_compiled()
    old = ext.backward_mode()
    ext.set_backward_mode(mode)
    try:
        for name, (ad, ai, ap, (r, c)), (bd, bi, bp, _) in _pairs(dtype):
            ext.clear_plan_cache()
            ai, ap, bi, bp = (np.asarray(v, np.int64) for v in (ai, ap, bi, bp))
            AI, AP, BI, BP = to_dev(dev, ai, ap, bi, bp)
            shared = None
            built0 = ext.plan_cache_stats()[0]
            for it, (alpha, beta) in enumerate(((1.0, 1.0), (1.0, -1.0), (0.75, -2.5), (-0.5, 3.0))):
                a_vals = (ad * (1 + it)).astype(dtype) + randn(20 + it, ad.shape[0], dtype)
                b_vals = (bd * (2 - it)).astype(dtype) + randn(30 + it, bd.shape[0], dtype)
                Cd_ref, Ci_ref, Cp_ref = oracle.splincomb_forward(r, c, alpha, a_vals, ai, ap, beta, b_vals, bi, bp)
                AD, BD = to_dev(dev, a_vals, b_vals)
                Cd, Ci, Cp = ext.splincomb_forward(r, c, torch.tensor(alpha), AD, AI, AP, torch.tensor(beta), BD, BI, BP)
                assert_same(host(Cp), Cp_ref, f"{name} call {it} C_indptr")
                assert_same(host(Ci), Ci_ref, f"{name} call {it} C_indices")
                assert_same(host(Cd), Cd_ref, f"{name} call {it} C_data")
                g = randn(3 + it, Cd_ref.shape[0], dtype)
                gA, gB = ext.splincomb_backward(r, c, torch.tensor(alpha), AD, AI, AP, torch.tensor(beta), BD, BI, BP,
                                                to_dev(dev, g)[0], Ci, Cp)
                gA_ref, gB_ref = oracle.splincomb_backward(r, c, alpha, a_vals, ai, ap, beta, b_vals, bi, bp, g,
                                                           Ci_ref, Cp_ref)
                assert_same(host(gA), gA_ref, f"{name} call {it} grad_A")
                assert_same(host(gB), gB_ref, f"{name} call {it} grad_B")
                # a backward given a copy of the pattern (not the tensors the plan handed out) must
                # not trust the maps' positions blindly: it searches, with the same result
                gA2, gB2 = ext.splincomb_backward(r, c, torch.tensor(alpha), AD, AI, AP, torch.tensor(beta), BD, BI,
                                                  BP, to_dev(dev, g)[0], Ci.clone(), Cp.clone())
                assert_same(host(gA2), gA_ref, f"{name} call {it} grad_A on a copied pattern")
                assert_same(host(gB2), gB_ref, f"{name} call {it} grad_B on a copied pattern")
                first_planned = 2 if mode == "planned" else 1
                if Cd_ref.shape[0] > 0 and it >= first_planned:
                    # results on the maps share the plan's pattern tensors
                    if shared is not None:
                        assert Ci.data_ptr() == shared[0] and Cp.data_ptr() == shared[1], f"{name} call {it}"
                    shared = (Ci.data_ptr(), Cp.data_ptr())
            if Cd_ref.shape[0] > 0:
                assert ext.plan_cache_stats()[0] - built0 == 1, f"{name}: one set of maps for the pair"
    finally:
        ext.set_backward_mode(old)
        ext.clear_plan_cache()


def test_splincomb_maps_at_full_size(dev):
    # the 2048 x 2048 Poisson pattern (4.2 M rows) against a shifted copy of itself: the pass over the
    # cached maps and the gathering backward give the bits of the merging forward and the searching
    # backward, and (A - B) + B has A's pattern again with values equal to rounding
    ext = numml_amd.load_compiled()
    old = ext.backward_mode()
    d, i, p, (r, c) = G.poisson2d(2048, np.float32, jitter_seed=0)
    d2 = G.poisson2d(2048, np.float32, jitter_seed=1)[0]
    AD, BD, I, P = to_dev(dev, d, d2, i, p)
    BI, BP = I.clone(), P.clone()
    g = to_dev(dev, randn(4, d.shape[0], np.float32))[0]
    one, mone = torch.tensor(1.0), torch.tensor(-1.0)
    try:
        ext.set_backward_mode("atomic")
        ref = ext.splincomb_forward(r, c, one, AD, I, P, mone, BD, BI, BP)
        gref = ext.splincomb_backward(r, c, one, AD, I, P, mone, BD, BI, BP, g, ref[1], ref[2])
        ext.set_backward_mode("eager")
        ext.clear_plan_cache()
        ext.splincomb_forward(r, c, one, AD, I, P, mone, BD, BI, BP)          # records the maps
        out = ext.splincomb_forward(r, c, one, AD, I, P, mone, BD, BI, BP)    # runs on them
        gout = ext.splincomb_backward(r, c, one, AD, I, P, mone, BD, BI, BP, g, out[1], out[2])
        for a, b, what in zip(out + gout, ref + gref, ("C_data", "C_indices", "C_indptr", "grad_A", "grad_B")):
            assert torch.equal(a, b), what
        back = ext.splincomb_forward(r, c, one, out[0], out[1], out[2], one, BD, BI, BP)
        assert torch.equal(back[1], I) and torch.equal(back[2], P)
        assert_close(host(back[0]), d, "(A - B) + B")
    finally:
        ext.set_backward_mode(old)
        ext.clear_plan_cache()


@pytest.mark.parametrize("dtype", DTYPES)
def test_dense_rowsum_diagonal(dev, ext, dtype):
    cases = [("poisson", G.poisson2d(24, dtype, 1)), ("random", G.random_csr(130, 170, 0.07, 2, dtype)),
             ("tall", G.random_csr(400, 9, 0.3, 3, dtype)), ("one_dense_row", G.random_csr(3, 6000, 0.9, 4, dtype, empty_rows=False)),
             ("powerlaw", G.powerlaw(2500, 2500, 30000, max_deg=2000, seed=5, dtype=dtype)),
             ("empty", (np.zeros(0, dtype), np.zeros(0, np.int64), np.zeros(5, np.int64), (4, 4)))]
    for name, (d, i, p, (r, c)) in cases:
        D, I, P = to_dev(dev, d, i, p)
        if r * c <= 4_000_000:
            Ad = ext.csr_to_dense_forward(r, c, D, I, P)
            assert_same(host(Ad), oracle.csr_to_dense_forward(r, c, d, i, p), f"{name} dense")
            gD = randn(1, (r, c), dtype)
            assert_same(host(ext.csr_to_dense_backward(to_dev(dev, gD)[0], r, c, D, I, P)),
                        oracle.csr_to_dense_backward(gD, r, c, d, i, p), f"{name} dense backward")
            wide = to_dev(dev, np.concatenate([gD, gD], axis=1))[0][:, :c]          # row stride 2c
            assert_same(host(ext.csr_to_dense_backward(wide, r, c, D, I, P)),
                        oracle.csr_to_dense_backward(gD, r, c, d, i, p), f"{name} dense backward, strided")
        rs = ext.csr_row_sum_forward(r, c, D, I, P)
        rs_ref = oracle.csr_row_sum_forward(r, c, d, i, p)
        if int(np.diff(p).max(initial=0)) <= 512:
            assert_same(host(rs), rs_ref, f"{name} row sums")
        else:
            assert_close(host(rs), rs_ref, f"{name} row sums")
        g = randn(2, r, dtype)
        Gv = to_dev(dev, g)[0]
        assert_same(host(ext.csr_row_sum_backward(Gv, r, c, D, I, P)), oracle.csr_row_sum_backward(g, r, c, d, i, p),
                    f"{name} row sum backward")
        if r <= c:                                                     # x has one entry per row
            assert_same(host(ext.csr_extract_diagonal_forward(r, c, D, I, P)),
                        oracle.csr_extract_diagonal_forward(r, c, d, i, p), f"{name} diagonal")
            assert_same(host(ext.csr_extract_diagonal_backward(Gv, r, c, D, I, P)),
                        oracle.csr_extract_diagonal_backward(g, r, c, d, i, p), f"{name} diagonal backward")


def test_operators_and_gradients(dev):
    ad, ai, ap, (n, _) = G.poisson2d(12, np.float64, 1)
    bd, bi, bp, _ = G.tridiag(n, np.float64)
    A = sp.SparseCSRTensor(tuple(to_dev(dev, ad, ai, ap)), (n, n))
    B = sp.SparseCSRTensor(tuple(to_dev(dev, bd, bi, bp)), (n, n))
    A.requires_grad = True
    B.requires_grad = True
    Ad, Bd = A.to_dense().detach(), B.to_dense().detach()
    assert torch.equal((A + B).to_dense(), Ad + Bd)                       # numml/tests/test_splincomb.py pattern
    assert torch.equal((A - B).to_dense(), Ad - Bd)
    Z = A - A
    assert Z.nnz == A.nnz and not bool(Z.data.any())                     # explicit zeros are kept
    assert torch.equal((2.0 * A).to_dense(), 2.0 * Ad) and torch.equal((-A).to_dense(), -Ad)
    assert torch.equal(abs(-A).data, A.data.abs()) and torch.equal((A ** 2).data, A.data ** 2)
    # loss through +, row_sum, diagonal and to_dense
    w = to_dev(dev, randn(1, n, np.float64))[0]
    loss = ((A - B).row_sum() * w).sum() + (A + B).diagonal().sum() + (A.to_dense() ** 2).sum() + A.trace()
    loss.backward()
    rows_a = A.row_indices
    rows_b = B.row_indices
    gA = w[rows_a] + (A.indices == rows_a) * 2.0 + 2 * A.data.detach()
    gB = -w[rows_b] + (B.indices == rows_b) * 1.0
    assert torch.allclose(A.data.grad, gA, atol=1e-12) and torch.allclose(B.data.grad, gB, atol=1e-12)
    with pytest.raises(RuntimeError, match="Incompatible shapes"):
        A + sp.eye(3, dtype=torch.float64, device=dev)
    assert torch.equal(A.sum(), A.data.sum())


def test_triangles_and_diagonal_index(dev):
    import scipy.sparse as sps
    d, i, p, (n, _) = G.poisson2d(9, np.float64, 2)
    A = sp.SparseCSRTensor(tuple(to_dev(dev, d, i, p)), (n, n))
    A.requires_grad = True
    S = sps.csr_matrix((d, i, p), shape=(n, n))
    for k in (-1, 0, 2):
        for mine, theirs in ((A.tril(k), sps.tril(S, k).tocsr()), (A.triu(k), sps.triu(S, k).tocsr())):
            theirs.sort_indices()
            assert_same(host(mine.indptr), theirs.indptr.astype(np.int64), "indptr")
            assert_same(host(mine.indices), theirs.indices.astype(np.int64), "indices")
            assert_same(host(mine.data), theirs.data, "data")
    # a solve with the lower triangle, differentiated back to A: entries above the diagonal get zero
    b = to_dev(dev, randn(1, n, np.float64))[0]
    x = A.tril().solve_triangular(upper=False, unit=False, b=b)
    x.sum().backward()
    upper = A.indices > A.row_indices
    assert not bool(A.data.grad[upper].any()) and bool(A.data.grad[~upper].any())
    rows = np.repeat(np.arange(n), np.diff(p))
    want = np.full(n, -1, np.int64)
    want[rows[i == rows]] = np.nonzero(i == rows)[0]
    assert_same(host(A.diagonal_idx), want, "diagonal_idx")
