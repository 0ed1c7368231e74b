"""Product plan of a sparse product (nm_spgemm_plan_build and the kernels that run on it).

The planned numeric product and the mapped gradients must reproduce, bit for bit, what the
stateless SpGEMM kernels and the CPU oracle give (whose sums run in the order of
cpp/sparse_csr_cpu.cpp:177-303): structure is exact, values are compared with assert_same.
"""
import numpy as np
import pytest
import torch

import oracle
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as mirror
from util import assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]


def _short_rows(rows, cols, max_len, seed, dtype, min_len=0):
    return G.ragged_csr(rows, cols, max_len, seed, dtype, min_len=min_len)


def _cases(dtype):
    yield "poisson2d x poisson2d", G.poisson2d(23, dtype, jitter_seed=1), G.poisson2d(23, dtype, jitter_seed=2)
    yield "laplace3d x laplace3d", G.laplace3d(9, dtype, jitter_seed=3), G.laplace3d(9, dtype, jitter_seed=4)
    yield "tridiag x tridiag", G.tridiag(300, dtype), G.tridiag(300, dtype)
    a = _short_rows(500, 300, 8, 5, dtype)
    b = _short_rows(300, 700, 8, 6, dtype)
    yield "ragged rectangular, empty rows", a, b
    a = _short_rows(64, 40, 8, 7, dtype, min_len=8)
    b = _short_rows(40, 4000, 8, 8, dtype, min_len=8)
    yield "every row full: 64 entries per row of C", a, b
    a = _short_rows(1, 1, 1, 9, dtype, min_len=1)
    yield "one by one", a, a


def _unpack(m):
    d, i, p = m[0], m[1], m[2]
    shape = m[3] if len(m) > 3 else None
    return d, i, p, shape


@pytest.mark.parametrize("dtype", DTYPES)
def test_planned_product_and_gradients_match_the_stateless_kernels_and_the_oracle(dev, dtype):
    for name, A, B in _cases(dtype):
        ad, ai, ap, ashape = _unpack(A)
        bd, bi, bp, bshape = _unpack(B)
        A_rows, A_cols = ashape
        B_rows, B_cols = bshape
        assert A_cols == B_rows, name
        AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
        C_data, C_indices, C_indptr = mirror.spgemm_forward(A_rows, A_cols, AD, AI, AP, B_rows, B_cols, BD, BI, BP)
        plan = mirror.ProductPlan(A_rows, A_cols, AI, AP, BI, BP, C_indices, C_indptr)
        assert plan.usable, name
        # new values on the same patterns: the plan knows nothing of the values it was built beside
        ad2, bd2 = randn(11, ad.shape[0], dtype), randn(12, bd.shape[0], dtype)
        AD2, BD2 = to_dev(dev, ad2, bd2)
        ref_data, ref_indices, ref_indptr = mirror.spgemm_forward(A_rows, A_cols, AD2, AI, AP, B_rows, B_cols, BD2,
                                                                  BI, BP)
        assert_same(host(ref_indices), host(C_indices), f"{name}: pattern")
        got = plan.numeric(AD2, BD2)
        assert_same(host(got), host(ref_data), f"{name}: C_data vs stateless kernels")
        cd, ci, cp = oracle.spgemm_forward(A_rows, A_cols, ad2, ai, ap, B_rows, B_cols, bd2, bi, bp)
        assert_same(host(got), cd, f"{name}: C_data vs oracle")
        g = randn(13, cd.shape[0], dtype)
        Gz, = to_dev(dev, g)
        gA, gB = plan.backward(Gz, AD2, BD2)
        rA, rB = oracle.spgemm_backward(g, ci, cp, A_rows, A_cols, ad2, ai, ap, B_rows, B_cols, bd2, bi, bp)
        assert_same(host(gA), rA, f"{name}: grad_A vs oracle")
        assert_same(host(gB), rB, f"{name}: grad_B vs oracle")
        # the same product computed on the records its own symbolic phase leaves behind, and the plan
        # those records make
        md, mi, mp, mplan = mirror.spgemm_forward_mapped(A_rows, A_cols, AD2, AI, AP, B_rows, B_cols, BD2, BI, BP)
        assert_same(host(mp), cp, f"{name}: C_indptr (mapped forward)")
        assert_same(host(mi), ci, f"{name}: C_indices (mapped forward)")
        assert_same(host(md), cd, f"{name}: C_data (mapped forward)")
        assert mplan.usable, name
        assert_same(host(mplan.numeric(AD, BD)), host(C_data), f"{name}: C_data on the adopted plan")
        mA, mB = mplan.backward(Gz, AD2, BD2)
        assert_same(host(mA), rA, f"{name}: grad_A on the adopted plan")
        assert_same(host(mB), rB, f"{name}: grad_B on the adopted plan")
        old = mirror.BACKWARD_MODE
        mirror.BACKWARD_MODE = "eager"
        try:
            sA, sB = mirror.spgemm_backward(Gz, C_indices, C_indptr, A_rows, A_cols, AD2, AI, AP, B_rows, B_cols,
                                            BD2, BI, BP)
        finally:
            mirror.BACKWARD_MODE = old
        assert_same(host(gA), host(sA), f"{name}: grad_A vs the search-based kernel")
        assert_same(host(gB), host(sB), f"{name}: grad_B vs the search-based kernel")


def test_backward_walks_far_reaching_patterns_in_strips(dev):
    """When A reaches 8192 rows or more from its diagonal, the kernel that forms both gradients walks
    each XCD's share of the rows in strips.  The order is only a schedule: every row must still be
    taken exactly once.  A band at +-9000 on 300 000 rows leaves a tail that the strips do not cover
    (walked in plain order), and one gradient alone still goes through the two separate kernels."""
    import scipy.sparse as sps
    n, far = 300_000, 9000
    rng = np.random.default_rng(3)
    diags = [rng.standard_normal(n - abs(o)) for o in (-far, -1, 0, 1, far)]
    A = sps.diags(diags, (-far, -1, 0, 1, far), shape=(n, n), format="csr")
    A.sort_indices()
    ad, ai, ap = A.data.copy(), A.indices.astype(np.int64), A.indptr.astype(np.int64)
    bd = rng.standard_normal(ad.shape[0])
    AD, AI, AP, BD = to_dev(dev, ad, ai, ap, bd)
    C_data, C_indices, C_indptr = mirror.spgemm_forward(n, n, AD, AI, AP, n, n, BD, AI, AP)
    plan = mirror.ProductPlan(n, n, AI, AP, AI, AP, C_indices, C_indptr)
    assert plan.usable
    cd, ci, cp = oracle.spgemm_forward(n, n, ad, ai, ap, n, n, bd, ai, ap)
    assert_same(host(plan.numeric(AD, BD)), cd, "C_data")
    g = randn(5, cd.shape[0], np.float64)
    Gz, = to_dev(dev, g)
    rA, rB = oracle.spgemm_backward(g, ci, cp, n, n, ad, ai, ap, n, n, bd, ai, ap)
    gA, gB = plan.backward(Gz, AD, BD)
    assert_same(host(gA), rA, "grad_A (both gradients in one walk, in strips)")
    assert_same(host(gB), rB, "grad_B (both gradients in one walk, in strips)")


def test_signed_zeros_and_explicit_zeros_keep_the_serial_result(dev):
    dtype = np.float64
    ad, ai, ap, ashape = _unpack(G.poisson2d(12, dtype))
    bd, bi, bp, bshape = _unpack(G.poisson2d(12, dtype))
    ad = ad.copy()
    bd = bd.copy()
    ad[::3] = 0.0
    ad[1::7] = -0.0
    bd[::4] = -1.0
    bd[2::5] = 0.0
    n = ashape[0]
    AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
    C_data, C_indices, C_indptr = mirror.spgemm_forward(n, n, AD, AI, AP, n, n, BD, BI, BP)
    plan = mirror.ProductPlan(n, n, AI, AP, BI, BP, C_indices, C_indptr)
    assert plan.usable
    got = plan.numeric(AD, BD)
    cd, ci, cp = oracle.spgemm_forward(n, n, ad, ai, ap, n, n, bd, bi, bp)
    assert np.array_equal(np.signbit(host(got)), np.signbit(cd)), "signs of zeros"
    assert_same(host(got), cd, "C_data")


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_rows_of_the_left_operand_and_wide_rows_of_the_product(dev, dtype):
    """Classes 2 and 3 of the plan: rows of A of any length (products that take the hash path), rows
    of C of up to 254 entries; B's named rows stay within eight entries."""
    cases = [
        ("(A A) A on a 3D grid: 25-entry rows of A, 62-entry rows of C", 2, None),
        ("ragged rows of up to 30 entries times rows of up to 8: wide rows of C", 3,
         (G.ragged_csr(700, 500, 30, 61, dtype), G.ragged_csr(500, 90000, 8, 62, dtype, min_len=4))),
        ("ragged rows of up to 30 entries times rows of up to 2", 2,
         (G.ragged_csr(900, 800, 30, 63, dtype, min_len=9), G.ragged_csr(800, 50, 2, 64, dtype))),
    ]
    for name, want_class, mats in cases:
        if mats is None:
            d, i, p, (n, _) = G.laplace3d(12, dtype, jitter_seed=5)
            D, I, P = to_dev(dev, d, i, p)
            Ld, Li, Lp = mirror.spgemm_forward(n, n, D, I, P, n, n, D, I, P)
            A = (host(Ld), host(Li), host(Lp), (n, n))
            B = (d, i, p, (n, n))
        else:
            A, B = mats
        ad, ai, ap, (m, kdim) = A
        bd, bi, bp, (_, ncols) = B
        AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
        C_data, C_indices, C_indptr = mirror.spgemm_forward(m, kdim, AD, AI, AP, kdim, ncols, BD, BI, BP)
        plan = mirror.ProductPlan(m, kdim, AI, AP, BI, BP, C_indices, C_indptr)
        assert plan.usable and plan.plan_class == want_class, (name, plan.plan_class)
        ad2, bd2 = randn(71, ad.shape[0], dtype), randn(72, bd.shape[0], dtype)
        AD2, BD2 = to_dev(dev, ad2, bd2)
        cd, ci, cp = oracle.spgemm_forward(m, kdim, ad2, ai, ap, kdim, ncols, bd2, bi, bp)
        assert_same(host(C_indices), ci, f"{name}: pattern")
        assert_same(host(plan.numeric(AD2, BD2)), cd, f"{name}: C_data")
        g = randn(73, cd.shape[0], dtype)
        gA, gB = plan.backward(to_dev(dev, g)[0], AD2, BD2)
        rA, rB = oracle.spgemm_backward(g, ci, cp, m, kdim, ad2, ai, ap, kdim, ncols, bd2, bi, bp)
        assert_same(host(gA), rA, f"{name}: grad_A")
        assert_same(host(gB), rB, f"{name}: grad_B")


@pytest.mark.parametrize("dtype", DTYPES)
def test_named_rows_of_the_right_operand_of_up_to_32_entries(dev, dtype):
    """Classes 4 to 7 of the plan: two or four destination octets per entry of A, for products whose
    rows of B have up to 16 or 32 entries (a 3D stencil times its own square, a 27-point matrix
    squared).  Product and both gradients bit for bit, as for the one-octet plans."""
    def stencil27(n):
        import scipy.sparse as sps
        one = sps.diags([np.ones(n - 1), np.ones(n), np.ones(n - 1)], [-1, 0, 1])
        M = sps.kron(sps.kron(one, one), one).tocsr()
        M.sort_indices()
        rng = np.random.default_rng(7)
        return (rng.standard_normal(M.nnz).astype(dtype), M.indices.astype(np.int64), M.indptr.astype(np.int64), M.shape)

    d, i, p, (n, _) = G.laplace3d(10, dtype, jitter_seed=5)
    D, I, P = to_dev(dev, d, i, p)
    Sd, Si, Sp = mirror.spgemm_forward(n, n, D, I, P, n, n, D, I, P)
    square = (host(Sd), host(Si), host(Sp), (n, n))
    cases = [
        ("rows of up to 6 entries times rows of 9 to 16", 4,
         G.ragged_csr(600, 500, 6, 81, dtype, min_len=1), G.ragged_csr(500, 3000, 16, 82, dtype, min_len=9)),
        ("rows of up to 7 entries times rows of 17 to 32", 5,
         G.ragged_csr(400, 300, 7, 83, dtype), G.ragged_csr(300, 9000, 32, 84, dtype, min_len=17)),
        ("rows of up to 12 entries times rows of up to 20", 5,
         G.ragged_csr(700, 500, 12, 85, dtype, min_len=5), G.ragged_csr(500, 600, 20, 86, dtype, min_len=3)),
        ("A (A A) on a 3D grid: 25-entry rows of B, 63-entry rows of C", 5, (d, i, p, (n, n)), square),
        ("27-point matrix squared: 27-entry rows of B, 125-entry rows of C", 5, stencil27(9), stencil27(9)),
    ]
    for name, want_class, A, B in cases:
        ad, ai, ap, (m, kdim) = A
        bd, bi, bp, (_, ncols) = B
        AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
        C_data, C_indices, C_indptr = mirror.spgemm_forward(m, kdim, AD, AI, AP, kdim, ncols, BD, BI, BP)
        plan = mirror.ProductPlan(m, kdim, AI, AP, BI, BP, C_indices, C_indptr)
        # 4 / 5: two / four octets; 6 / 7: the same with rows of C of more than 64 entries
        want = want_class + (2 if int(np.diff(host(C_indptr)).max()) > 64 else 0)
        assert plan.usable and plan.plan_class == want, (name, plan.plan_class, want)
        ad2, bd2 = randn(91, ad.shape[0], dtype), randn(92, bd.shape[0], dtype)
        AD2, BD2 = to_dev(dev, ad2, bd2)
        cd, ci, cp = oracle.spgemm_forward(m, kdim, ad2, ai, ap, kdim, ncols, bd2, bi, bp)
        assert_same(host(C_indices), ci, f"{name}: pattern")
        assert_same(host(plan.numeric(AD2, BD2)), cd, f"{name}: C_data")
        g = randn(93, cd.shape[0], dtype)
        gA, gB = plan.backward(to_dev(dev, g)[0], AD2, BD2)
        rA, rB = oracle.spgemm_backward(g, ci, cp, m, kdim, ad2, ai, ap, kdim, ncols, bd2, bi, bp)
        assert_same(host(gA), rA, f"{name}: grad_A")
        assert_same(host(gB), rB, f"{name}: grad_B")
        # one gradient at a time
        L = mirror._lib.lib()
        for which in (0, 1):
            out = torch.full_like(AD2 if which == 0 else BD2, 7.0)
            mirror._lib.check(L.nm_spgemm_backward_mapped_wide(
                mirror._dt(AD2), plan.plan_class, m, kdim, ad.shape[0], bd.shape[0], cd.shape[0],
                mirror._ptr(to_dev(dev, g)[0]), mirror._ptr(AD2), mirror._ptr(plan.transposed.mem), mirror._ptr(BD2),
                mirror._ptr(BP), mirror._ptr(plan.mem), mirror._ptr(out) if which == 0 else None,
                mirror._ptr(out) if which == 1 else None, mirror._stream(dev)), "nm_spgemm_backward_mapped_wide")
            assert_same(host(out), rA if which == 0 else rB, f"{name}: gradient {which} alone")


def test_rows_beyond_the_limits_are_refused(dev):
    dtype = np.float64
    # a row of C with more than 254 entries
    ad, ai, ap, ashape = _unpack(_short_rows(50, 60, 40, 21, dtype, min_len=40))
    bd, bi, bp, bshape = _unpack(_short_rows(60, 80000, 8, 22, dtype, min_len=8))
    AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
    _, C_indices, C_indptr = mirror.spgemm_forward(50, 60, AD, AI, AP, 60, 80000, BD, BI, BP)
    assert int((C_indptr[1:] - C_indptr[:-1]).max()) > 254
    assert not mirror.ProductPlan(50, 60, AI, AP, BI, BP, C_indices, C_indptr).usable
    # a named row of B with 33 entries (up to 32 there are plans with two or four octets per entry)
    ad, ai, ap, ashape = _unpack(_short_rows(50, 60, 4, 23, dtype, min_len=1))
    bd, bi, bp, bshape = _unpack(_short_rows(60, 800, 33, 24, dtype, min_len=33))
    AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
    _, C_indices, C_indptr = mirror.spgemm_forward(50, 60, AD, AI, AP, 60, 800, BD, BI, BP)
    plan = mirror.ProductPlan(50, 60, AI, AP, BI, BP, C_indices, C_indptr)
    assert not plan.usable
    with pytest.raises(RuntimeError):
        plan.numeric(AD, BD)
    # a pattern of C that is not the product's
    ad, ai, ap, ashape = _unpack(G.tridiag(40, dtype))
    AD, AI, AP = to_dev(dev, ad, ai, ap)
    assert not mirror.ProductPlan(40, 40, AI, AP, AI, AP, AI, AP).usable


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("dtype", DTYPES)
def test_random_short_row_products(dev, seed, dtype):
    """Shapes, fill and row lengths drawn at random inside the plan's limits (rows of 0..8 entries in
    both operands, rectangular, columns never named, rows never named)."""
    rng = np.random.default_rng(100 + seed)
    m, kdim, n = (int(rng.integers(1, 3000)) for _ in range(3))
    la, lb = int(rng.integers(1, 9)), int(rng.integers(1, 9))
    ad, ai, ap, _ = G.ragged_csr(m, kdim, min(la, kdim), 200 + seed, dtype)
    bd, bi, bp, _ = G.ragged_csr(kdim, n, min(lb, n), 300 + seed, dtype)
    AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
    C_data, C_indices, C_indptr = mirror.spgemm_forward(m, kdim, AD, AI, AP, kdim, n, BD, BI, BP)
    plan = mirror.ProductPlan(m, kdim, AI, AP, BI, BP, C_indices, C_indptr)
    if ai.shape[0] == 0:
        assert not plan.usable          # nothing to plan for a matrix without entries
        return
    assert plan.usable
    md, mi, mp, mplan = mirror.spgemm_forward_mapped(m, kdim, AD, AI, AP, kdim, n, BD, BI, BP)
    assert_same(host(mi), host(C_indices), "pattern (mapped forward)")
    assert_same(host(md), host(C_data), "C_data (mapped forward)")
    assert mplan.usable
    # the adopted plan is the built one, array for array (flag word, then bstart, cstart, dest,
    # each starting on a multiple of 256 bytes)
    nnz_a, off = ai.shape[0], 256
    for name, width in (("bstart", 4), ("cstart", 4), ("dest", 8)):
        assert torch.equal(mplan.mem[off:off + nnz_a * width], plan.mem[off:off + nnz_a * width]), name
        off += ((nnz_a + 1) * width + 255) // 256 * 256
    ad2, bd2 = randn(seed, ad.shape[0], dtype), randn(seed + 50, bd.shape[0], dtype)
    AD2, BD2 = to_dev(dev, ad2, bd2)
    cd, ci, cp = oracle.spgemm_forward(m, kdim, ad2, ai, ap, kdim, n, bd2, bi, bp)
    assert_same(host(C_indices), ci, "pattern")
    assert_same(host(plan.numeric(AD2, BD2)), cd, "C_data")
    g = randn(seed + 70, cd.shape[0], dtype)
    gA, gB = plan.backward(to_dev(dev, g)[0], AD2, BD2)
    rA, rB = oracle.spgemm_backward(g, ci, cp, m, kdim, ad2, ai, ap, kdim, n, bd2, bi, bp)
    assert_same(host(gA), rA, "grad_A")
    assert_same(host(gB), rB, "grad_B")
