"""Pins the CPU oracle (oracle/) three ways, without a GPU:

1. against fixtures written from the reference's own compiled CPU sources
   (tests/golden/hotpath_golden.npz, made by tests/golden/make_golden.py);
2. against that compiled reference directly, when oracle/_ref is present;
3. against what the mathematics fixes: dense products, SciPy's product of the
   patterns, closed-form gradients (numml/tests/test_spmv.py:62-107,
   test_spdmm.py:58-113, test_spmm.py:69-110), residuals and known inverses
   (test_sptrsv.py:11-110).

Every comparison with the reference's code is bitwise.
"""
import importlib.util
import os

import numpy as np
import pytest
import scipy.sparse as sp
import scipy.sparse.linalg as spla

import oracle
from numml_amd import generators as G
from oracle import ref

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
make_golden = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_golden)

GOLD = np.load(os.path.join(HERE, "golden", "hotpath_golden.npz"))
CASES = make_golden.cases()


def same(a, b, what):
    assert a.dtype == b.dtype and a.shape == b.shape, what
    assert np.array_equal(a, b, equal_nan=True), f"{what}: differs bitwise"


# ------------------------------------------------------------------ golden fixtures

@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_golden_products(tag):
    m = CASES[f"mat_{tag}"]
    (ad, ai, ap, (ar, ac)), (bd, bi, bp, (br, bc)) = m["A"], m["B"]
    same(oracle.spgemv_forward(ar, ac, ad, ai, ap, m["x"]), GOLD[f"{tag}_spgemv_y"], "spgemv y")
    gA, gx = oracle.spgemv_backward(m["g"], ar, ac, ad, ai, ap, m["x"])
    same(gA, GOLD[f"{tag}_spgemv_gA"], "spgemv grad_A")
    same(gx, GOLD[f"{tag}_spgemv_gx"], "spgemv grad_x")
    same(oracle.spdmm_forward(ar, ac, ad, ai, ap, m["Bd"]), GOLD[f"{tag}_spdmm_C"], "spdmm C")
    gA, gB = oracle.spdmm_backward(ar, ac, ad, ai, ap, m["Bd"], m["gC"])
    same(gA, GOLD[f"{tag}_spdmm_gA"], "spdmm grad_A")
    same(gB, GOLD[f"{tag}_spdmm_gB"], "spdmm grad_B")
    Cd, Ci, Cp = oracle.spgemm_forward(ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
    same(Cp, GOLD[f"{tag}_spgemm_Cp"], "spgemm indptr")
    same(Ci, GOLD[f"{tag}_spgemm_Ci"], "spgemm indices")
    same(Cd, GOLD[f"{tag}_spgemm_Cd"], "spgemm data")
    gA, gB = oracle.spgemm_backward(GOLD[f"{tag}_spgemm_gC"], Ci, Cp, ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
    same(gA, GOLD[f"{tag}_spgemm_gA"], "spgemm grad_A")
    same(gB, GOLD[f"{tag}_spgemm_gB"], "spgemm grad_B")
    pd_, pi, pp, (pr, pc) = m["P"]
    Cd, Ci, Cp = oracle.spgemm_forward(pr, pc, pd_, pi, pp, pr, pc, pd_, pi, pp)
    same(Cp, GOLD[f"{tag}_spgemm_PP_Cp"], "P@P indptr")
    same(Ci, GOLD[f"{tag}_spgemm_PP_Ci"], "P@P indices")
    same(Cd, GOLD[f"{tag}_spgemm_PP_Cd"], "P@P data")
    T = oracle.csr_transpose(ar, ac, ad, ai, ap)
    for name, v in zip(("d", "i", "p", "perm"), T):
        same(v, GOLD[f"{tag}_transpose_{name}"], f"transpose {name}")


@pytest.mark.parametrize("tag", ["f32", "f64"])
@pytest.mark.parametrize("lower", [True, False])
@pytest.mark.parametrize("unit", [False, True])
def test_golden_sptrsv(tag, lower, unit):
    t = CASES[f"tri_{tag}"][lower]
    ld, li, lp, (n, _) = t["L"]
    key = f"{tag}_sptrsv_{'lo' if lower else 'up'}_{'unit' if unit else 'diag'}"
    x = oracle.sptrsv_forward(n, n, ld, li, lp, lower, unit, t["b"])
    same(x, GOLD[key + "_x"], "x")
    gA, gb = oracle.sptrsv_backward(t["g"], x, n, n, ld, li, lp, lower, unit)
    # stored entries on the wrong side of the diagonal, and the diagonal of a unit solve,
    # still get -grad_b[i] * x[j] (cpp/sparse_csr_cpu.cpp:750-755)
    same(gA, GOLD[key + "_gA"], "grad_A")
    same(gb, GOLD[key + "_gb"], "grad_b")


def test_golden_explicit_zero_is_kept():
    (ad, ai, ap, (ar, ac)), (bd, bi, bp, (br, bc)) = CASES["cancel"]["A"], CASES["cancel"]["B"]
    Cd, Ci, Cp = oracle.spgemm_forward(ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
    same(Cp, GOLD["cancel_Cp"], "indptr")
    same(Ci, GOLD["cancel_Ci"], "indices")
    same(Cd, GOLD["cancel_Cd"], "data")
    assert Cd.tolist() == [0.0] and Cp.tolist() == [0, 1]   # 1*1 + 1*(-1): stored although zero


# ------------------------------------------------------------- compiled reference

needs_ref = pytest.mark.skipif(not ref.built(), reason="oracle/_ref not built (needs the reference tree)")


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_ref_products(dtype, seed):
    rng = np.random.default_rng(100 + seed)
    r, k, c = (int(v) for v in rng.integers(1, 90, 3))
    A = G.random_csr(r, k, float(rng.uniform(0.02, 0.3)), 10 * seed, dtype)
    B = G.random_csr(k, c, float(rng.uniform(0.02, 0.3)), 10 * seed + 1, dtype)
    (ad, ai, ap, _), (bd, bi, bp, _) = A, B
    x, g = rng.standard_normal(k).astype(dtype), rng.standard_normal(r).astype(dtype)
    same(oracle.spgemv_forward(r, k, ad, ai, ap, x), ref.call("spgemv_forward", r, k, ad, ai, ap, x), "y")
    for a, b in zip(oracle.spgemv_backward(g, r, k, ad, ai, ap, x),
                    ref.call("spgemv_backward", g, r, k, ad, ai, ap, x)):
        same(a, b, "spgemv backward")
    Bd, gC = rng.standard_normal((k, 9)).astype(dtype), rng.standard_normal((r, 9)).astype(dtype)
    same(oracle.spdmm_forward(r, k, ad, ai, ap, Bd), ref.call("spdmm_forward", r, k, ad, ai, ap, Bd), "C")
    for a, b in zip(oracle.spdmm_backward(r, k, ad, ai, ap, Bd, gC),
                    ref.call("spdmm_backward", r, k, ad, ai, ap, Bd, gC)):
        same(a, b, "spdmm backward")
    C1 = oracle.spgemm_forward(r, k, ad, ai, ap, k, c, bd, bi, bp)
    C2 = ref.call("spgemm_forward", r, k, ad, ai, ap, k, c, bd, bi, bp)
    for a, b in zip(C1, C2):
        same(a, b, "spgemm forward")
    gCs = rng.standard_normal(C1[0].shape[0]).astype(dtype)
    for a, b in zip(oracle.spgemm_backward(gCs, C1[1], C1[2], r, k, ad, ai, ap, k, c, bd, bi, bp),
                    ref.call("spgemm_backward", gCs, C1[1], C1[2], r, k, ad, ai, ap, k, c, bd, bi, bp)):
        same(a, b, "spgemm backward")
    T1 = oracle.csr_transpose(r, k, ad, ai, ap)
    for a, b in zip(T1, ref.call("csr_transpose_forward", r, k, ad, ai, ap)):
        same(a, b, "transpose")
    gT = rng.standard_normal(ad.shape[0]).astype(dtype)
    same(oracle.csr_transpose_backward(gT, T1[3]), ref.call("csr_transpose_backward", gT, T1[3]),
         "transpose backward")
    # the transpose of the transpose is the matrix itself; its permutation undoes the first
    T2 = oracle.csr_transpose(k, r, T1[0], T1[1], T1[2])
    same(T2[0], ad, "(A^T)^T data"), same(T2[1], ai, "(A^T)^T indices"), same(T2[2], ap, "(A^T)^T indptr")
    same(T1[3][T2[3]], np.arange(ad.shape[0]), "permutations compose to the identity")


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("lower", [True, False])
@pytest.mark.parametrize("unit", [False, True])
def test_ref_sptrsv(dtype, lower, unit):
    for seed, wrong in ((1, 0.0), (2, 0.02)):
        ld, li, lp, (n, _) = G.random_tri(120, 0.06, seed, lower, dtype, wrong_side=wrong)
        rng = np.random.default_rng(seed)
        b, g = rng.standard_normal(n).astype(dtype), rng.standard_normal(n).astype(dtype)
        x = oracle.sptrsv_forward(n, n, ld, li, lp, lower, unit, b)
        same(x, ref.call("sptrsv_forward", n, n, ld, li, lp, lower, unit, b), "x")
        for a, c in zip(oracle.sptrsv_backward(g, x, n, n, ld, li, lp, lower, unit),
                        ref.call("sptrsv_backward", g, x, n, n, ld, li, lp, lower, unit, b)):
            same(a, c, "sptrsv backward")


# -------------------------------------------------------------------- mathematics

def _dense(csr):
    d, i, p, shape = csr
    return sp.csr_matrix((d, i, p), shape=shape).toarray()


def test_math_spmv_and_gradients():
    d, i, p, (n, _) = G.tridiag(64, np.float64)
    A = _dense((d, i, p, (n, n)))
    for j in (0, 17, 63):                      # unit vectors return columns (test_spmv.py:21-39)
        e = np.zeros(n)
        e[j] = 1.0
        assert np.array_equal(oracle.spgemv_forward(n, n, d, i, p, e), A[:, j])
    assert not oracle.spgemv_forward(n, n, d, i, p, np.zeros(n)).any()
    rng = np.random.default_rng(0)
    x, g = rng.standard_normal(n), rng.standard_normal(n)
    np.testing.assert_allclose(oracle.spgemv_forward(n, n, d, i, p, x), A @ x, rtol=1e-13, atol=1e-13)
    gA, gx = oracle.spgemv_backward(g, n, n, d, i, p, x)
    rows = np.repeat(np.arange(n), np.diff(p))
    assert np.array_equal(gA, g[rows] * x[i])                    # grad_A[k] = g[row] x[col]
    np.testing.assert_allclose(gx, A.T @ g, rtol=1e-13, atol=1e-13)


def test_math_spdmm_and_gradients():
    csr = G.random_csr(50, 40, 0.1, 3, np.float64)
    d, i, p, (r, c) = csr
    A = _dense(csr)
    rng = np.random.default_rng(1)
    B, gC = rng.standard_normal((c, 6)), rng.standard_normal((r, 6))
    np.testing.assert_allclose(oracle.spdmm_forward(r, c, d, i, p, B), A @ B, rtol=1e-12, atol=1e-13)
    gA, gB = oracle.spdmm_backward(r, c, d, i, p, B, gC)
    rows = np.repeat(np.arange(r), np.diff(p))
    np.testing.assert_allclose(gA, (gC @ B.T)[rows, i], rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(gB, A.T @ gC, rtol=1e-12, atol=1e-13)


def test_math_spgemm_structure_values_gradients():
    A, B = G.random_csr(60, 45, 0.08, 5, np.float64), G.random_csr(45, 70, 0.08, 6, np.float64)
    (ad, ai, ap, (ar, ac)), (bd, bi, bp, (br, bc)) = A, B
    Cd, Ci, Cp = oracle.spgemm_forward(ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
    # structure = product of the patterns (no cancellation), columns ascending
    pat = sp.csr_matrix((np.ones_like(ad), ai, ap), shape=(ar, ac)) @ \
        sp.csr_matrix((np.ones_like(bd), bi, bp), shape=(br, bc))
    pat.sort_indices()
    assert np.array_equal(Cp, pat.indptr) and np.array_equal(Ci, pat.indices)
    Ad, Bd = _dense(A), _dense(B)
    rows = np.repeat(np.arange(ar), np.diff(Cp))
    np.testing.assert_allclose(Cd, (Ad @ Bd)[rows, Ci], rtol=1e-12, atol=1e-13)
    gC = np.random.default_rng(2).standard_normal(Cd.shape[0])
    gCd = np.zeros((ar, bc))
    gCd[rows, Ci] = gC
    gA, gB = oracle.spgemm_backward(gC, Ci, Cp, ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
    arow, brow = np.repeat(np.arange(ar), np.diff(ap)), np.repeat(np.arange(br), np.diff(bp))
    np.testing.assert_allclose(gA, (gCd @ Bd.T)[arow, ai], rtol=1e-12, atol=1e-13)   # (gC B^T) on mask(A)
    np.testing.assert_allclose(gB, (Ad.T @ gCd)[brow, bi], rtol=1e-12, atol=1e-13)   # (A^T gC) on mask(B)


def test_math_laplace3d_square_has_25_per_interior_row():
    d, i, p, (n, _) = G.laplace3d(9, np.float64, jitter_seed=0)
    Cd, Ci, Cp = oracle.spgemm_forward(n, n, d, i, p, n, n, d, i, p)
    per_row = np.diff(Cp).reshape(9, 9, 9)
    assert (per_row[2:-2, 2:-2, 2:-2] == 25).all() and per_row.max() == 25
    for r in range(n):
        assert np.all(np.diff(Ci[Cp[r]:Cp[r + 1]]) > 0)


@pytest.mark.parametrize("lower", [True, False])
@pytest.mark.parametrize("unit", [False, True])
def test_math_sptrsv(lower, unit):
    csr = G.random_tri(80, 0.08, 7, lower, np.float64)
    d, i, p, (n, _) = csr
    T = _dense(csr)
    if unit:
        np.fill_diagonal(T, 1.0)
    rng = np.random.default_rng(3)
    b, g = rng.standard_normal(n), rng.standard_normal(n)
    x = oracle.sptrsv_forward(n, n, d, i, p, lower, unit, b)
    np.testing.assert_allclose(T @ x, b, rtol=1e-10, atol=1e-10)          # residual (test_sptrsv.py:27-110)
    np.testing.assert_allclose(x, spla.spsolve_triangular(sp.csr_matrix(T), b, lower=lower), rtol=1e-9, atol=1e-10)
    gA, gb = oracle.sptrsv_backward(g, x, n, n, d, i, p, lower, unit)
    np.testing.assert_allclose(T.T @ gb, g, rtol=1e-10, atol=1e-10)       # grad_b = T^{-T} g
    rows = np.repeat(np.arange(n), np.diff(p))
    assert np.array_equal(gA, -(gb[rows] * x[i]))                          # -grad_b x^T on the mask


def test_math_identity_and_bidiagonal_solves():
    n = 50
    eye = (np.ones(n), np.arange(n, dtype=np.int64), np.arange(n + 1, dtype=np.int64))
    b = np.random.default_rng(4).standard_normal(n)
    assert np.array_equal(oracle.sptrsv_forward(n, n, *eye, True, False, b), b)      # test_sptrsv.py:11-25
    d, i, p, _ = G.bidiag(n, np.float64, lower=True)       # 2I - E_-1: x_k = sum_j b_j / 2^(k-j+1)
    x = oracle.sptrsv_forward(n, n, d, i, p, True, False, b)
    closed = np.array([sum(b[j] / 2.0 ** (k - j + 1) for j in range(k + 1)) for k in range(n)])
    np.testing.assert_allclose(x, closed, rtol=1e-13, atol=1e-13)


def test_math_fp32_solve_accumulates_in_double():
    # rounding happens once at the end (cpp/sparse_csr_cpu.cpp:659-662, :722)
    csr = G.random_tri(200, 0.05, 9, True, np.float32)
    d, i, p, (n, _) = csr
    b = np.random.default_rng(5).standard_normal(n).astype(np.float32)
    x32 = oracle.sptrsv_forward(n, n, d, i, p, True, False, b)
    x64 = oracle.sptrsv_forward(n, n, d.astype(np.float64), i, p, True, False, b.astype(np.float64))
    assert x32.dtype == np.float32 and np.array_equal(x32, x64.astype(np.float32))


def test_generators_match_the_stated_sizes():
    d, i, p, (n, _) = G.poisson2d(256)
    assert n == 65536 and d.shape[0] == 326656 and d.dtype == np.float64
    assert set(np.unique(d)) == {-1.0, 4.0}
    d, i, p, (n, _) = G.laplace3d(16)
    assert d.shape[0] == 7 * 16 ** 3 - 6 * 16 ** 2
    d, i, p, (n, _) = G.poisson2d_lower(32)
    assert d.shape[0] == 3 * 32 * 32 - 2 * 32 and np.all((d[p[1:] - 1] >= 4) & (d[p[1:] - 1] < 5))
    d, i, p, (r, c) = G.powerlaw(5000, 5000, 80000, seed=0)
    lens = np.diff(p)
    assert lens.min() >= 1 and abs(d.shape[0] - 80000) < 20000
    for row in range(0, r, 97):
        assert np.all(np.diff(i[p[row]:p[row + 1]]) > 0)
    np.testing.assert_allclose(np.add.reduceat(d.astype(np.float64), p[:-1]), 1.0, rtol=1e-5)


# ------------------------------------------------- entrywise / reduction operations

def _pair(dtype, seed):
    """Two matrices of one shape with overlapping patterns (some rows empty in either)."""
    rng = np.random.default_rng(300 + seed)
    r, c = (int(v) for v in rng.integers(1, 70, 2))
    A = G.random_csr(r, c, float(rng.uniform(0.05, 0.4)), 20 * seed, dtype)
    B = G.random_csr(r, c, float(rng.uniform(0.05, 0.4)), 20 * seed + 1, dtype)
    return r, c, A[:3], B[:3]


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_ref_lincomb_and_reductions(dtype, seed):
    r, c, (ad, ai, ap), (bd, bi, bp) = _pair(dtype, seed)
    alpha, beta = np.array(0.75, dtype), np.array(-1.5, dtype)
    C1 = oracle.splincomb_forward(r, c, float(alpha), ad, ai, ap, float(beta), bd, bi, bp)
    C2 = ref.call("splincomb_forward", r, c, alpha, ad, ai, ap, beta, bd, bi, bp)
    for a, b, what in zip(C1, C2, ("C_data", "C_indices", "C_indptr")):
        same(a, b, f"splincomb {what}")
    gC = np.random.default_rng(seed).standard_normal(C1[0].shape[0]).astype(dtype)
    for a, b in zip(oracle.splincomb_backward(r, c, float(alpha), ad, ai, ap, float(beta), bd, bi, bp, gC, C1[1], C1[2]),
                    ref.call("splincomb_backward", r, c, alpha, ad, ai, ap, beta, bd, bi, bp, gC, C1[1], C1[2])):
        same(a, b, "splincomb backward")
    same(oracle.csr_to_dense_forward(r, c, ad, ai, ap), ref.call("csr_to_dense_forward", r, c, ad, ai, ap), "to_dense")
    gD = np.random.default_rng(seed + 1).standard_normal((r, c)).astype(dtype)
    same(oracle.csr_to_dense_backward(gD, r, c, ad, ai, ap),
         ref.call("csr_to_dense_backward", gD, r, c, ad, ai, ap), "to_dense backward")
    same(oracle.csr_row_sum_forward(r, c, ad, ai, ap), ref.call("csr_row_sum_forward", r, c, ad, ai, ap), "row_sum")
    g = np.random.default_rng(seed + 2).standard_normal(r).astype(dtype)
    same(oracle.csr_row_sum_backward(g, r, c, ad, ai, ap),
         ref.call("csr_row_sum_backward", g, r, c, ad, ai, ap), "row_sum backward")
    n = min(r, c)                                   # the diagonal ops index x by row: square part only
    sq = sp.csr_matrix((ad, ai, ap), shape=(r, c))[:n, :n].tocsr()
    sq.sort_indices()
    sd, si, sp_ = sq.data.astype(dtype), sq.indices.astype(np.int64), sq.indptr.astype(np.int64)
    same(oracle.csr_extract_diagonal_forward(n, n, sd, si, sp_),
         ref.call("csr_extract_diagonal_forward", n, n, sd, si, sp_), "diagonal")
    same(oracle.csr_extract_diagonal_backward(g[:n], n, n, sd, si, sp_),
         ref.call("csr_extract_diagonal_backward", g[:n], n, n, sd, si, sp_), "diagonal backward")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_math_lincomb_and_reductions(dtype):
    r, c, (ad, ai, ap), (bd, bi, bp) = _pair(dtype, 5)
    Ad = sp.csr_matrix((ad, ai, ap), shape=(r, c)).toarray()
    Bd = sp.csr_matrix((bd, bi, bp), shape=(r, c)).toarray()
    Cd, Ci, Cp = oracle.splincomb_forward(r, c, 2.0, ad, ai, ap, -3.0, bd, bi, bp)
    # structure: union of the patterns (SciPy sum of the all-ones matrices has no cancellation)
    U = sp.csr_matrix((np.ones_like(ad), ai, ap), shape=(r, c)) + sp.csr_matrix((np.ones_like(bd), bi, bp), shape=(r, c))
    U.sort_indices()
    assert np.array_equal(Cp, U.indptr) and np.array_equal(Ci, U.indices)
    assert np.array_equal(sp.csr_matrix((Cd, Ci, Cp), shape=(r, c)).toarray(), (dtype(2.0) * Ad + dtype(-3.0) * Bd))
    # A - A keeps explicit zeros on A's pattern
    Zd, Zi, Zp = oracle.splincomb_forward(r, c, 1.0, ad, ai, ap, -1.0, ad, ai, ap)
    assert np.array_equal(Zi, ai) and np.array_equal(Zp, ap) and not Zd.any()
    # gradients: d(sum(w . C))/dA[k] = alpha * w at A's column, same for B with beta
    w = np.random.default_rng(1).standard_normal(Cd.shape[0]).astype(dtype)
    gA, gB = oracle.splincomb_backward(r, c, 2.0, ad, ai, ap, -3.0, bd, bi, bp, w, Ci, Cp)
    W = sp.csr_matrix((w, Ci, Cp), shape=(r, c)).toarray()
    rows_a, rows_b = np.repeat(np.arange(r), np.diff(ap)), np.repeat(np.arange(r), np.diff(bp))
    assert np.array_equal(gA, W[rows_a, ai] * dtype(2.0)) and np.array_equal(gB, W[rows_b, bi] * dtype(-3.0))
    # dense round trip, row sums, diagonal
    assert np.array_equal(oracle.csr_to_dense_forward(r, c, ad, ai, ap), Ad)
    assert np.array_equal(oracle.csr_to_dense_backward(Ad, r, c, ad, ai, ap), ad)
    rs = oracle.csr_row_sum_forward(r, c, ad, ai, ap)
    assert np.allclose(rs, Ad.sum(axis=1), rtol=1e-5 if dtype == np.float32 else 1e-12, atol=1e-6)
    g = np.random.default_rng(2).standard_normal(r).astype(dtype)
    assert np.array_equal(oracle.csr_row_sum_backward(g, r, c, ad, ai, ap), g[rows_a])
    n = min(r, c)
    td, ti, tp, _ = G.poisson2d(6, dtype, 3)
    assert np.array_equal(oracle.csr_extract_diagonal_forward(36, 36, td, ti, tp),
                          sp.csr_matrix((td, ti, tp), shape=(36, 36)).diagonal())
    gd = oracle.csr_extract_diagonal_backward(g[:1].repeat(36), 36, 36, td, ti, tp)
    on_diag = ti == np.repeat(np.arange(36), np.diff(tp))
    assert np.array_equal(gd, np.where(on_diag, g[0], 0).astype(dtype))
    sd, si, sp_, _ = G.random_csr(9, 9, 0.3, 1, dtype)       # some rows without a stored diagonal
    assert np.array_equal(oracle.csr_extract_diagonal_forward(9, 9, sd, si, sp_),
                          sp.csr_matrix((sd, si, sp_), shape=(9, 9)).diagonal())


# ------------------------------------------------------------------ sparse LU

def _lu_cases(dtype):
    yield "tridiag", G.tridiag(12, dtype)
    yield "poisson6", G.poisson2d(6, dtype, 1)
    rng = np.random.default_rng(5)
    n = 40
    m = sp.random(n, n, 0.08, random_state=3, format="csr", dtype=np.float64) + sp.eye(n) * 4.0
    m = m.tocsr()
    m.sort_indices()
    yield "random_diag_dominant", (m.data.astype(dtype), m.indices.astype(np.int64), m.indptr.astype(np.int64), (n, n))
    a = sp.random(25, 25, 0.1, random_state=7, format="csr", dtype=np.float64)
    a = (a + a.T + sp.eye(25) * 6.0).tocsr()
    a.sort_indices()
    yield "symmetric_pattern", (a.data.astype(dtype), a.indices.astype(np.int64), a.indptr.astype(np.int64), (25, 25))


@needs_ref
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_ref_splu_and_spsolve_backward(dtype):
    for name, (d, i, p, (n, _)) in _lu_cases(dtype):
        mine = oracle.splu(n, n, d, i, p)
        theirs = ref.call("splu", n, n, d, i, p)
        for a, b, what in zip(mine, theirs, ("M_data", "M_indices", "M_indptr", "Mt_data", "Mt_indices", "Mt_indptr")):
            same(a, b, f"{name} splu {what}")
        rng = np.random.default_rng(1)
        gx, x = rng.standard_normal(n).astype(dtype), rng.standard_normal(n).astype(dtype)
        for a, b in zip(oracle.spsolve_backward(gx, x, n, n, mine[3], mine[4], mine[5], d, i, p),
                        ref.call("spsolve_backward", gx, x, n, n, mine[3], mine[4], mine[5], d, i, p)):
            same(a, b, f"{name} spsolve_backward")


def test_math_splu_factors_reproduce_the_matrix():
    for name, (d, i, p, (n, _)) in _lu_cases(np.float64):
        Md, Mi, Mp, Td, Ti, Tp = oracle.splu(n, n, d, i, p)
        M = sp.csr_matrix((Md, Mi, Mp), shape=(n, n)).toarray()
        L, U = np.tril(M, -1) + np.eye(n), np.triu(M)
        A = sp.csr_matrix((d, i, p), shape=(n, n)).toarray()
        assert np.allclose(L @ U, A, atol=1e-10), name
        assert np.array_equal(sp.csr_matrix((Td, Ti, Tp), shape=(n, n)).toarray(), M.T), name
        # the filled pattern contains A's and is what symbolic elimination of the pattern gives
        pat = (A != 0)
        for k in range(n):
            rows_k = np.nonzero(pat[k + 1:, k])[0] + k + 1
            cols_k = np.nonzero(pat[k, k + 1:])[0] + k + 1
            pat[np.ix_(rows_k, cols_k)] = True
        assert np.array_equal(sp.csr_matrix((np.ones_like(Md), Mi, Mp), shape=(n, n)).toarray() != 0, pat), name
        # a solve through the factors
        b = np.random.default_rng(2).standard_normal(n)
        y = oracle.sptrsv_forward(n, n, Md, Mi, Mp, True, True, b)
        x = oracle.sptrsv_forward(n, n, Md, Mi, Mp, False, False, y)
        assert np.allclose(A @ x, b, atol=1e-9), name
