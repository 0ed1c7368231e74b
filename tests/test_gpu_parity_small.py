"""HIP kernels (through the C ABI) against the serial oracle on small seeded inputs.

Covers the shapes the reference's tests use (1-D Poisson N=16/2048,
numml/tests/test_spmv.py:9-10) plus empty rows, empty matrices, ragged and long
rows, both dtypes, both triangles, unit and non-unit diagonals.
"""
import numpy as np
import pytest
import scipy.sparse as sps
import torch

import oracle
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as ext
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

# products none of whose rows of B is handed to the workgroup-per-row kernel (row length x column
# length of A at most 4096): the planned backward adds grad_B in the serial order
EXACT_GRAD_B = {"stencil_25x7", "stencil_7x25", "stencil_25x25", "all_le_8", "a_le_10_b_le_10", "full_8",
                "narrow_b", "one_row", "empty"}

DTYPES = [np.float32, np.float64]


def _matrices(dtype):
    yield "tridiag16", G.tridiag(16, dtype)
    yield "tridiag2048", G.tridiag(2048, dtype)
    yield "poisson64", G.poisson2d(64, dtype, jitter_seed=3)
    yield "random_ragged", G.random_csr(700, 300, 0.02, 5, dtype)
    yield "one_dense_row", G.random_csr(40, 5000, 0.9, 6, dtype, empty_rows=False)
    yield "powerlaw", G.powerlaw(3000, 3000, target_nnz=60000, max_deg=2500, seed=7, dtype=dtype)
    # 20-30 entries in every row: a block of rows does not fit LDS and is taken in runs of rows
    yield "ragged_25", G.ragged_csr(2000, 1500, 30, 8, dtype, min_len=20)
    yield "empty", (np.zeros(0, dtype), np.zeros(0, np.int64), np.zeros(6, np.int64), (5, 4))


@pytest.fixture(params=["planned", "atomic"])
def backward_mode(request):
    old = ext.BACKWARD_MODE
    ext.BACKWARD_MODE = request.param
    yield request.param
    ext.BACKWARD_MODE = old


STENCILS = ("tridiag16", "tridiag2048", "poisson64")


@pytest.mark.parametrize("dtype", DTYPES)
def test_spmv_forward_backward(dev, dtype, backward_mode):
    for name, (d, i, p, (rows, cols)) in _matrices(dtype):
        x, g = randn(1, cols, dtype), randn(2, rows, dtype)
        y_ref = oracle.spgemv_forward(rows, cols, d, i, p, x)
        gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
        D, I, P, X, Gd = to_dev(dev, d, i, p, x, g)
        y = ext.spgemv_forward(rows, cols, D, I, P, X)
        gA, gx = ext.spgemv_backward(Gd, rows, cols, D, I, P, X)
        assert_close(host(y), y_ref, f"{name} y")
        assert_same(host(gA), gA_ref, f"{name} grad_A")
        assert_close(host(gx), gx_ref, f"{name} grad_x")
        if name in STENCILS or name == "ragged_25":
            # short rows are summed in storage order: bit-identical to the serial loop
            assert_same(host(y), y_ref, f"{name} y (bitwise)")
        if name in STENCILS and backward_mode == "planned":
            # columns are summed in ascending row order as well
            assert_same(host(gx), gx_ref, f"{name} grad_x (bitwise)")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 7, 64, 100])
def test_spmm_forward_backward(dev, dtype, n, backward_mode):
    for name, (d, i, p, (rows, cols)) in _matrices(dtype):
        if name == "one_dense_row" and n > 7:
            continue
        B, gC = randn(1, (cols, n), dtype), randn(2, (rows, n), dtype)
        C_ref = oracle.spdmm_forward(rows, cols, d, i, p, B)
        gA_ref, gB_ref = oracle.spdmm_backward(rows, cols, d, i, p, B, gC)
        D, I, P, Bd, gCd = to_dev(dev, d, i, p, B, gC)
        C = ext.spdmm_forward(rows, cols, D, I, P, Bd)
        gA, gB = ext.spdmm_backward(rows, cols, D, I, P, Bd, gCd)
        # rows up to 512 entries are summed in storage order (bitwise); longer rows are shared
        # by eight wavefronts and match to rounding
        if int(np.diff(p).max(initial=0)) <= 512:
            assert_same(host(C), C_ref, f"{name} C")
        else:
            assert_close(host(C), C_ref, f"{name} C")
        assert_close(host(gA), gA_ref, f"{name} grad_A")
        assert_close(host(gB), gB_ref, f"{name} grad_B")
        if backward_mode == "planned" and int(np.bincount(i, minlength=1).max()) <= 512:
            assert_same(host(gB), gB_ref, f"{name} grad_B (bitwise)")


@pytest.mark.parametrize("dtype", DTYPES)
def test_spmm_backward_on_one_walk(dev, dtype):
    """The backward on a plan forms both gradients in one walk over A by column.  Against the oracle, and bit for bit against the two separate walks it replaces (the C
    ABI computes one gradient alone the old way), on patterns with columns of more than 512
    entries (shared by a workgroup), empty columns and rows, and a single long chunk."""
    import ctypes
    import scipy.sparse as sps
    from numml_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(5)

    def with_dense_columns(rows, cols, density, dense_cols):
        M = sps.random(rows, cols, density=density, random_state=7, format="lil", dtype=np.float64)
        for c in dense_cols:
            M[:, c] = rng.standard_normal((rows, 1))
        M = M.tocsr().astype(dtype)
        M.sort_indices()
        return M.data.copy(), M.indices.astype(np.int64), M.indptr.astype(np.int64), (rows, cols)

    cases = [("ragged", G.random_csr(700, 300, 0.02, 5, dtype)),
             ("long_columns", with_dense_columns(1500, 200, 0.01, (3, 77, 199))),
             ("one_column", with_dense_columns(900, 1, 0.0, (0,))),
             ("powerlaw_T", G.powerlaw(3000, 3000, target_nnz=60000, max_deg=2500, seed=7, dtype=dtype)),
             ("poisson64", G.poisson2d(64, dtype, jitter_seed=3))]
    # the power-law matrix transposed: its long rows become long columns
    d, i, p, (r, c) = cases[3][1]
    T = sps.csr_matrix((d, i, p), shape=(r, c)).T.tocsr()
    T.sort_indices()
    cases[3] = ("powerlaw_T", (T.data.astype(dtype), T.indices.astype(np.int64), T.indptr.astype(np.int64), (c, r)))
    old = ext.BACKWARD_MODE
    ext.BACKWARD_MODE = "eager"
    try:
        for name, (d, i, p, (rows, cols)) in cases:
            for n in (5, 33, 64, 100):
                B, gC = randn(1, (cols, n), dtype), randn(2, (rows, n), dtype)
                gA_ref, gB_ref = oracle.spdmm_backward(rows, cols, d, i, p, B, gC)
                D, I, P, Bd, gCd = to_dev(dev, d, i, p, B, gC)
                gA, gB = ext.spdmm_backward(rows, cols, D, I, P, Bd, gCd)
                assert_close(host(gA), gA_ref, f"{name} n={n} grad_A")
                assert_close(host(gB), gB_ref, f"{name} n={n} grad_B")
                longest = int(np.bincount(i, minlength=1).max()) if i.size else 0
                if longest <= 512:
                    assert_same(host(gB), gB_ref, f"{name} n={n} grad_B (bitwise)")
                # one gradient at a time goes the old way: the row-major dot products, the product on the plan
                plan = ext._transpose_plan(I, P, rows, cols, dev)
                gA2, gB2 = torch.empty_like(D), torch.empty_like(gB)
                args = (ext._dt(D), rows, cols, D.shape[0], D.data_ptr(), I.data_ptr(), P.data_ptr(),
                        plan.mem.data_ptr(), Bd.data_ptr(), n, gCd.data_ptr(), n, n)
                assert L.nm_spdmm_backward_planned(*args, gA2.data_ptr(), None, n, None) == 0
                assert L.nm_spdmm_backward_planned(*args, None, gB2.data_ptr(), n, None) == 0
                torch.cuda.synchronize()
                if longest <= 512 and n > 32:
                    assert_same(host(gA), host(gA2), f"{name} n={n} grad_A: one walk vs two")
                    assert_same(host(gB), host(gB2), f"{name} n={n} grad_B: one walk vs two")
                elif longest <= 512:    # up to 32 columns the separate dot products fold 8-32 lanes, not 64
                    assert_close(host(gA), host(gA2), f"{name} n={n} grad_A: one walk vs two")
                    assert_same(host(gB), host(gB2), f"{name} n={n} grad_B: one walk vs two")
                else:       # columns shared by a workgroup sum their dot products in another order
                    assert_close(host(gA), host(gA2), f"{name} n={n} grad_A: one walk vs two")
                    assert_same(host(gB), host(gB2), f"{name} n={n} grad_B: one walk vs two")
    finally:
        ext.BACKWARD_MODE = old


def test_spmm_strided_operand(dev):
    d, i, p, (rows, cols) = G.random_csr(200, 150, 0.05, 11, np.float64)
    wide = randn(3, (cols, 40), np.float64)
    D, I, P, W = to_dev(dev, d, i, p, wide)
    C = ext.spdmm_forward(rows, cols, D, I, P, W[:, 4:20])          # row stride 40, 16 columns
    Ct = ext.spdmm_forward(rows, cols, D, I, P, W[:, ::2])           # column stride 2 -> copied
    assert_same(host(C), oracle.spdmm_forward(rows, cols, d, i, p, wide[:, 4:20]), "strided rows")
    assert_same(host(Ct), oracle.spdmm_forward(rows, cols, d, i, p, wide[:, ::2]), "strided columns")


def test_spmm_thousands_of_dense_columns(dev, backward_mode):
    """A dense operand wider than one workgroup's slice of columns (1024) and than the widest the
    one-walk backward takes (4096): the forward and the product of the backward are cut into
    slices over the grid, the dot products of grad_A are shared by a workgroup's wavefronts.
    Against cpp/sparse_csr_cpu.cpp:599-646."""
    mode = backward_mode
    dtype, n = np.float64, 4200
    d, i, p, (rows, cols) = G.random_csr(150, 90, 0.08, 21, dtype)
    B, gC = randn(5, (cols, n), dtype), randn(6, (rows, n), dtype)
    C_ref = oracle.spdmm_forward(rows, cols, d, i, p, B)
    gA_ref, gB_ref = oracle.spdmm_backward(rows, cols, d, i, p, B, gC)
    D, I, P, Bd, gCd = to_dev(dev, d, i, p, B, gC)
    for sighting in range(2):   # (a plan is built at a pattern's second sighting)
        C = ext.spdmm_forward(rows, cols, D, I, P, Bd)
        gA, gB = ext.spdmm_backward(rows, cols, D, I, P, Bd, gCd)
        assert_same(host(C), C_ref, f"C ({mode}, call {sighting})")
        assert_close(host(gA), gA_ref, f"grad_A ({mode}, call {sighting})")
        assert_close(host(gB), gB_ref, f"grad_B ({mode}, call {sighting})")


@pytest.mark.parametrize("dtype", DTYPES)
def test_spgemm_forward_backward(dev, dtype):
    cases = [
        ("tridiag", G.tridiag(2048, dtype), G.tridiag(2048, dtype, 1.0, -2.0, 1.0)),
        ("poisson", G.poisson2d(48, dtype, 1), G.poisson2d(48, dtype, 2)),
        ("laplace3d", G.laplace3d(12, dtype, 0), G.laplace3d(12, dtype, 0)),
        ("rect", G.random_csr(300, 200, 0.03, 1, dtype), G.random_csr(200, 400, 0.04, 2, dtype)),
        ("dense_rows", G.random_csr(64, 600, 0.3, 3, dtype), G.random_csr(600, 900, 0.2, 4, dtype)),
        ("powerlaw", G.powerlaw(2000, 2000, 30000, max_deg=1500, seed=5, dtype=dtype),
         G.powerlaw(2000, 2000, 30000, max_deg=1500, seed=6, dtype=dtype)),
        ("spill", G.random_csr(6, 300, 0.9, 8, dtype, empty_rows=False),
         G.random_csr(300, 20000, 0.2, 9, dtype)),
        ("empty", (np.zeros(0, dtype), np.zeros(0, np.int64), np.zeros(4, np.int64), (3, 5)),
         G.random_csr(5, 6, 0.5, 1, dtype)),
    ]
    # rows of 25 and of 125 entries: the 16-lane bins of the hash path, columns that differ by
    # multiples of the grid's row and plane size, rows of C too long for the 8-lane backward
    a7 = G.laplace3d(16, dtype, 0)
    n3 = a7[3][0]
    a25 = oracle.spgemm_forward(n3, n3, *a7[:3], n3, n3, *a7[:3]) + ((n3, n3),)
    cases += [("stencil_25x7", a25, a7), ("stencil_7x25", a7, a25), ("stencil_25x25", a25, a25)]
    for name, (ad, ai, ap, (ar, ac)), (bd, bi, bp, (br, bc)) in cases:
        Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
        gC = randn(9, Cd_ref.shape[0], dtype)
        gA_ref, gB_ref = oracle.spgemm_backward(gC, Ci_ref, Cp_ref, ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
        AD, AI, AP, BD, BI, BP, GC = to_dev(dev, ad, ai, ap, bd, bi, bp, gC)
        Cd, Ci, Cp = ext.spgemm_forward(ar, ac, AD, AI, AP, br, bc, BD, BI, BP)
        assert_same(host(Cp), Cp_ref, f"{name} C_indptr")
        assert_same(host(Ci), Ci_ref, f"{name} C_indices")
        if name in ("spill",):
            assert_close(host(Cd), Cd_ref, f"{name} C_data")   # spilled rows add with atomics
        else:
            assert_same(host(Cd), Cd_ref, f"{name} C_data")
        for mode in ("planned", "atomic"):      # on the plan of A's pattern / stateless with atomics
            old_mode, ext.BACKWARD_MODE = ext.BACKWARD_MODE, mode
            try:
                gA, gB = ext.spgemm_backward(GC, Ci, Cp, ar, ac, AD, AI, AP, br, bc, BD, BI, BP)
            finally:
                ext.BACKWARD_MODE = old_mode
            assert_same(host(gA), gA_ref, f"{name} grad_A ({mode})")
            assert_close(host(gB), gB_ref, f"{name} grad_B ({mode})")
            if mode == "planned" and name in EXACT_GRAD_B:
                assert_same(host(gB), gB_ref, f"{name} grad_B ({mode}, bitwise)")


@pytest.mark.parametrize("dtype", DTYPES)
def test_spgemm_merge_path_over_many_workgroups(dev, dtype):
    """A stencil product large enough for thousands of workgroups whose wavefronts run out of
    step: the merge path's wavefronts share LDS arrays without a workgroup barrier, so each must
    keep to its own slots whatever the value type (fp32 rings once overlapped a neighbour's)."""
    d, i, p, (r, c) = G.laplace3d(40, dtype, 0)
    Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(r, c, d, i, p, r, c, d, i, p)
    D, I, P = to_dev(dev, d, i, p)
    for _ in range(3):
        Cd, Ci, Cp = ext.spgemm_forward(r, c, D, I, P, r, c, D, I, P)
        assert_same(host(Cp), Cp_ref, "C_indptr")
        assert_same(host(Ci), Ci_ref, "C_indices")
        assert_same(host(Cd), Cd_ref, "C_data")


@pytest.mark.parametrize("dtype", DTYPES)
def test_spgemm_mixed_short_and_long_rows(dev, dtype):
    """Rows that take the merge path (A row and its B rows of at most 8 entries) next to
    rows that do not, inside the same wavefront: lengths 0..8, exactly 8, 9 and longer."""
    cases = [
        ("all_le_8", G.ragged_csr(700, 500, 8, 1, dtype), G.ragged_csr(500, 600, 8, 2, dtype)),
        ("a_le_10_b_le_10", G.ragged_csr(1000, 400, 10, 3, dtype), G.ragged_csr(400, 450, 10, 4, dtype)),
        ("full_8", G.ragged_csr(300, 300, 8, 5, dtype, min_len=8), G.ragged_csr(300, 64, 8, 6, dtype, min_len=8)),
        ("b_long", G.ragged_csr(257, 100, 4, 7, dtype), G.ragged_csr(100, 3000, 40, 8, dtype)),
        ("narrow_b", G.ragged_csr(513, 90, 8, 9, dtype), G.ragged_csr(90, 3, 3, 10, dtype)),
        ("one_row", G.ragged_csr(1, 20, 8, 11, dtype, min_len=5), G.ragged_csr(20, 30, 8, 12, dtype)),
    ]
    for name, (ad, ai, ap, (ar, ac)), (bd, bi, bp, (br, bc)) in cases:
        Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
        gC = randn(9, Cd_ref.shape[0], dtype)
        gA_ref, gB_ref = oracle.spgemm_backward(gC, Ci_ref, Cp_ref, ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
        AD, AI, AP, BD, BI, BP, GC = to_dev(dev, ad, ai, ap, bd, bi, bp, gC)
        Cd, Ci, Cp = ext.spgemm_forward(ar, ac, AD, AI, AP, br, bc, BD, BI, BP)
        assert_same(host(Cp), Cp_ref, f"{name} C_indptr")
        assert_same(host(Ci), Ci_ref, f"{name} C_indices")
        assert_same(host(Cd), Cd_ref, f"{name} C_data")
        for mode in ("planned", "atomic"):      # on the plan of A's pattern / stateless with atomics
            old_mode, ext.BACKWARD_MODE = ext.BACKWARD_MODE, mode
            try:
                gA, gB = ext.spgemm_backward(GC, Ci, Cp, ar, ac, AD, AI, AP, br, bc, BD, BI, BP)
            finally:
                ext.BACKWARD_MODE = old_mode
            assert_same(host(gA), gA_ref, f"{name} grad_A ({mode})")
            assert_close(host(gB), gB_ref, f"{name} grad_B ({mode})")
            if mode == "planned" and name in EXACT_GRAD_B:
                assert_same(host(gB), gB_ref, f"{name} grad_B ({mode}, bitwise)")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lower", [True, False])
@pytest.mark.parametrize("unit", [False, True])
def test_sptrsv_forward_backward(dev, dtype, lower, unit):
    ext.clear_plan_cache()
    tri = lambda t: t if lower else _transpose(t)
    cases = [
        ("bidiag", G.bidiag(700, dtype, lower)),
        ("random", G.random_tri(400, 0.02, 3, lower, dtype)),
        ("random_wrong_side", G.random_tri(300, 0.03, 4, lower, dtype, wrong_side=0.01)),
        ("poisson_tri", tri(G.poisson2d_lower(40, dtype, 0))),
        ("wide_levels", G.random_tri(5000, 0.0004, 5, lower, dtype)),
        ("diag_only", G.random_tri(50, 0.0, 6, lower, dtype)),
    ]
    for name, case in cases:
        d, i, p, (n, _) = case
        b, g = randn(1, n, dtype), randn(2, n, dtype)
        x_ref = oracle.sptrsv_forward(n, n, d, i, p, lower, unit, b)
        gA_ref, gb_ref = oracle.sptrsv_backward(g, x_ref, n, n, d, i, p, lower, unit)
        D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
        x = ext.sptrsv_forward(n, n, D, I, P, lower, unit, Bv)
        assert_same(host(x), x_ref, f"{name} x")
        gA, gb = ext.sptrsv_backward(Gv, x, n, n, D, I, P, lower, unit, Bv)
        assert_same(host(gb), gb_ref, f"{name} grad_b")
        assert_same(host(gA), gA_ref, f"{name} grad_A")
    # 13 dependencies per row and levels of hundreds of rows (triangle of A @ A, 3D 7-point A):
    # the levels with thousands of entries get grid launches with 16 lanes per row, which add in
    # storage order; the small levels at both ends share rows among lanes and match to rounding
    a7 = G.laplace3d(56, dtype, 0)
    n = a7[3][0]
    Cd, Ci, Cp = oracle.spgemm_forward(n, n, *a7[:3], n, n, *a7[:3])
    M = sps.csr_matrix((Cd, Ci, Cp), shape=(n, n))
    # off-diagonal row sums below one, so that the unit-diagonal solve stays bounded
    M = (sps.tril(M, -1) if lower else sps.triu(M, 1)) * 0.01 + sps.diags(np.full(n, 1.25, dtype))
    M = M.tocsr().astype(dtype)
    M.sort_indices()
    d, i, p = M.data, M.indices.astype(np.int64), M.indptr.astype(np.int64)
    b, g = randn(1, n, dtype), randn(2, n, dtype)
    x_ref = oracle.sptrsv_forward(n, n, d, i, p, lower, unit, b)
    gA_ref, gb_ref = oracle.sptrsv_backward(g, x_ref, n, n, d, i, p, lower, unit)
    D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
    levels, launches = ext.sptrsv_schedule(n, I, P, lower)
    assert launches > 20, "levels with thousands of entries are expected to get launches of their own"
    x = ext.sptrsv_forward(n, n, D, I, P, lower, unit, Bv)
    assert_close(host(x), x_ref, "stencil triangle x")
    gA, gb = ext.sptrsv_backward(Gv, x, n, n, D, I, P, lower, unit, Bv)
    assert_close(host(gb), gb_ref, "stencil triangle grad_b")
    assert_close(host(gA), gA_ref, "stencil triangle grad_A")


def _transpose(csr):
    d, i, p, (r, c) = csr
    At_d, At_i, At_p, _ = oracle.csr_transpose(r, c, d, i, p)
    return At_d, At_i, At_p, (c, r)


def test_fp32_long_rows_against_a_double_evaluation(dev):
    # Long rows are summed by many lanes and reduced, i.e. in another order than the serial loop.
    # Both results are compared with the same products accumulated in double: the device's error
    # must not exceed four times the serial loop's, plus the fp32 tolerance of the parity rule.
    import scipy.sparse as sps
    rtol = 1e-5
    for name, (d, i, p, (rows, cols)) in (
            ("powerlaw", G.powerlaw(4000, 20000, target_nnz=400_000, max_deg=9000, seed=3, dtype=np.float32)),
            ("one_long_row", G.ragged_csr(3, 200_000, 150_000, 4, np.float32, min_len=100_000))):
        x = randn(1, cols, np.float32)
        B = randn(2, (cols, 8), np.float32)
        A64 = sps.csr_matrix((d.astype(np.float64), i, p), shape=(rows, cols))
        D, I, P, X, Bd = to_dev(dev, d, i, p, x, B)
        for what, got, cpu, exact in (
                ("spmv", host(ext.spgemv_forward(rows, cols, D, I, P, X)), oracle.spgemv_forward(rows, cols, d, i, p, x),
                 A64 @ x.astype(np.float64)),
                ("spmm", host(ext.spdmm_forward(rows, cols, D, I, P, Bd)), oracle.spdmm_forward(rows, cols, d, i, p, B),
                 A64 @ B.astype(np.float64))):
            err_gpu = np.abs(got.astype(np.float64) - exact)
            err_cpu = np.abs(cpu.astype(np.float64) - exact)
            bound = 4 * err_cpu + rtol * np.abs(exact).max()
            assert np.all(err_gpu <= bound), f"{name} {what}: worst excess {float((err_gpu - bound).max()):.3e}"


def test_sptrsv_signalling_equals_barriers_and_gives_up_instead_of_waiting_forever(dev):
    """The single-workgroup solve kernels can keep their wavefronts in step by neighbour-to-neighbour
    signals where the triangle allows it (a stencil's does) instead of a barrier per level.  Same
    bits either way; and with the poll limit forced from the host every wavefront leaves at once,
    the call returns, and x is NaN throughout instead of wrong."""
    import ctypes
    from numml_amd import _lib
    L = _lib.lib()
    d, i, p, (n, _) = G.poisson2d_lower(300, np.float64, diag_seed=2)      # 599 levels, up to 300 rows wide
    b = randn(3, n, np.float64)
    D, I, P, Bv = to_dev(dev, d, i, p, b)
    x_ref = oracle.sptrsv_forward(n, n, d, i, p, True, False, b)
    g = randn(4, n, np.float64)
    gA_ref, gb_ref = oracle.sptrsv_backward(g, x_ref, n, n, d, i, p, True, False)
    try:
        for signalling in (1, 0):
            assert L.nm_sptrsv_configure(0, signalling) == 0
            x = ext.sptrsv_forward(n, n, D, I, P, True, False, Bv)
            assert_same(host(x), x_ref, f"x (signalling={signalling})")
            gA, gb = ext.sptrsv_backward(to_dev(dev, g)[0], x, n, n, D, I, P, True, False, Bv)
            assert_same(host(gb), gb_ref, f"grad_b (signalling={signalling})")
            assert_same(host(gA), gA_ref, f"grad_A (signalling={signalling})")
        assert L.nm_sptrsv_configure(-1, 1) == 0                           # give up at once
        x = ext.sptrsv_forward(n, n, D, I, P, True, False, Bv)
        torch.cuda.synchronize()
        assert bool(torch.isnan(x).all())
    finally:
        assert L.nm_sptrsv_configure(0, 0) == 0
    x = ext.sptrsv_forward(n, n, D, I, P, True, False, Bv)
    assert_same(host(x), x_ref, "x after the defaults were restored")
