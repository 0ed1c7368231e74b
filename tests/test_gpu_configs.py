"""The five benchmark configurations at full size: HIP path against the serial
oracle on the same seeded inputs, plus size-independent identities.

Tolerance (fp32 1e-5, fp64 1e-12): |a - ref| <= rtol * |ref| + rtol * max|ref|;
SpGEMM structure and everything summed in the oracle's order is compared bitwise.
"""
import numpy as np
import pytest
import scipy.sparse as sps
import torch

import oracle
from numml_amd import _binding
from numml_amd import generators as G
from numml_amd import sparse as sp
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

ext = _binding.ops            # the binding the benchmark measures (the compiled one when it is built)


def test_cfg1_spmv_fp64_poisson256_autograd(dev):
    d, i, p, (rows, cols) = G.poisson2d(256, np.float64)
    x, g = randn(0, cols, np.float64), randn(1, rows, np.float64)
    D, I, P, X, Gv = to_dev(dev, d, i, p, x, g)
    A = sp.SparseCSRTensor((D, I, P), (rows, cols))
    A.requires_grad = True
    X.requires_grad_(True)
    y = A @ X
    y.backward(Gv)
    gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
    assert_same(host(y), oracle.spgemv_forward(rows, cols, d, i, p, x), "y")
    assert_same(host(A.data.grad), gA_ref, "grad_A")
    assert_same(host(X.grad), gx_ref, "grad_x")
    assert A.grad.shape == (rows, cols) and A.grad.nnz == d.shape[0]


@pytest.mark.parametrize("mode", ["eager", "atomic", "planned"])
def test_cfg2_spmv_fp32_poisson2048(dev, mode):
    d, i, p, (rows, cols) = G.poisson2d(2048, np.float32, jitter_seed=0)
    assert rows == 4194304 and d.shape[0] == 20963328
    x, g = randn(1, cols, np.float32), randn(2, rows, np.float32)
    D, I, P, X, Gv = to_dev(dev, d, i, p, x, g)
    ext.clear_plan_cache()
    _binding.set_backward_mode(mode)
    y = ext.spgemv_forward(rows, cols, D, I, P, X)
    gA, gx = ext.spgemv_backward(Gv, rows, cols, D, I, P, X)
    gA2, gx2 = ext.spgemv_backward(Gv, rows, cols, D, I, P, X)
    y2 = ext.spgemv_forward(rows, cols, D, I, P, X)      # in eager mode: through the plan's 32-bit structure
    assert torch.equal(y, y2)
    gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
    assert_same(host(y), oracle.spgemv_forward(rows, cols, d, i, p, x), "y")
    assert_same(host(gA), gA_ref, "grad_A")
    assert_close(host(gx), gx_ref, "grad_x")
    if mode == "eager":
        assert_same(host(gx), gx_ref, "grad_x (bitwise)")
        assert torch.equal(gx, gx2) and torch.equal(gA, gA2)       # run-to-run identical
    if mode == "planned":
        # the default mode: the first backward on the pattern ran the stateless kernels (atomic
        # sums, tolerance above); the second sighting built the plan and is the CPU loop's sum
        assert_same(host(gx2), gx_ref, "grad_x of the second backward (bitwise)")
        assert_same(host(gA2), gA_ref, "grad_A of the second backward")
        gA3, gx3 = ext.spgemv_backward(Gv, rows, cols, D, I, P, X)
        assert torch.equal(gx3, gx2) and torch.equal(gA3, gA2)
    # adjoint identity <A x, g> = <x, A^T g> in double
    lhs = float(host(y).astype(np.float64) @ g.astype(np.float64))
    rhs = float(host(gx).astype(np.float64) @ x.astype(np.float64))
    assert abs(lhs - rhs) <= 1e-5 * max(abs(lhs), 1.0) * 10


@pytest.mark.parametrize("mode", ["eager", "atomic", "planned"])
def test_cfg3_spmm_fp32_powerlaw(dev, mode):
    """eager: the fused kernel on the plan (what the benchmark times); atomic: the stateless
    kernels; planned (the default): stateless on the first backward of the pattern, on the plan from
    the second (the single-gradient calls at the end)."""
    rows = cols = 1_000_000
    n = 64
    d, i, p, _ = G.powerlaw(rows, cols, target_nnz=16_000_000, seed=0, dtype=np.float32)
    lens = np.diff(p)
    assert lens.max() == 10_000 and lens.min() >= 1 and 14e6 < d.shape[0] < 17e6
    B, gC = randn(1, (cols, n), np.float32), randn(2, (rows, n), np.float32)
    D, I, P, Bd, Gd = to_dev(dev, d, i, p, B, gC)
    ext.clear_plan_cache()
    _binding.set_backward_mode(mode)
    C = ext.spdmm_forward(rows, cols, D, I, P, Bd)
    gA, gB = ext.spdmm_backward(rows, cols, D, I, P, Bd, Gd)
    C, gA, gB = host(C), host(gA), host(gB)
    # every row of C against SciPy in double (rows of up to 10 000 entries included)
    A64 = sps.csr_matrix((d.astype(np.float64), i, p), shape=(rows, cols))
    C64 = A64 @ B.astype(np.float64)
    assert np.all(np.abs(C - C64) <= 1e-5 * np.abs(C64) + 1e-5 * np.abs(C64).max()), "C (all rows, vs double)"
    del C64
    # grad_A[k] = <gC[row(k)], B[col(k)]> (cpp/sparse_csr_cpu.cpp:625-636), EVERY stored entry, in
    # double, a million entries at a time
    row_of = np.repeat(np.arange(rows, dtype=np.int64), lens)
    want = np.empty(d.shape[0], np.float64)
    for k0 in range(0, d.shape[0], 1 << 20):
        k1 = min(k0 + (1 << 20), d.shape[0])
        want[k0:k1] = np.einsum("kn,kn->k", gC[row_of[k0:k1]].astype(np.float64), B[i[k0:k1]].astype(np.float64))
    assert np.all(np.abs(gA - want) <= 1e-5 * np.abs(want) + 1e-5 * np.abs(want).max()), "grad_A (all entries, vs double)"
    # oracle on the first 30k rows (its row->column->entry loop is slow): C and grad_A are row-local
    sub = 30_000
    nz = int(p[sub])
    C_ref = oracle.spdmm_forward(sub, cols, d[:nz], i[:nz], p[:sub + 1], B)
    gA_ref, _ = oracle.spdmm_backward(sub, cols, d[:nz], i[:nz], p[:sub + 1], B, gC[:sub])
    short = lens[:sub] <= 512          # summed in storage order: bitwise; longer rows: to rounding
    assert_same(C[:sub][short], C_ref[short], "C (first rows, short)")
    assert_close(C[:sub], C_ref, "C (first rows)")
    assert_close(gA[:nz], gA_ref, "grad_A (first rows)")
    # the longest row, wherever it is
    r = int(np.argmax(lens))
    sl = slice(int(p[r]), int(p[r + 1]))
    one = np.array([0, lens[r]], dtype=np.int64)
    assert_close(C[r:r + 1], oracle.spdmm_forward(1, cols, d[sl], i[sl], one, B), "C (longest row)")
    # grad_B = A^T gC against SciPy in double, all rows (cpp/sparse_csr_cpu.cpp:639-646)
    At = A64.T.tocsr()
    gB_ref = (At @ gC.astype(np.float64))
    scale = np.abs(gB_ref).max()
    assert np.all(np.abs(gB - gB_ref) <= 1e-5 * np.abs(gB_ref) + 1e-5 * scale)
    # adjoint identity <A B, gC> = <B, A^T gC>
    lhs = float(np.sum(C.astype(np.float64) * gC))
    rhs = float(np.sum(gB.astype(np.float64) * B))
    assert abs(lhs - rhs) <= 1e-4 * abs(lhs)
    # the gradient somebody asked for alone: the transposed product without the dot products
    # (the fixed adjacency of a GNN layer), and the dot products without the transposed product
    Breq = Bd.clone().requires_grad_(True)
    none_A, gB1 = ext.spdmm_backward(rows, cols, D, I, P, Breq, Gd)
    assert none_A is None
    if mode == "eager":
        assert_same(host(gB1), gB, "grad_B alone")
    else:
        assert np.all(np.abs(host(gB1) - gB_ref) <= 1e-5 * np.abs(gB_ref) + 1e-5 * scale), "grad_B alone"
    gA1, none_B = ext.spdmm_backward(rows, cols, D.clone().requires_grad_(True), I, P, Bd, Gd)
    assert none_B is None
    assert np.all(np.abs(host(gA1) - want) <= 1e-5 * np.abs(want) + 1e-5 * np.abs(want).max()), "grad_A alone"


def test_cfg4_spgemm_fp64_laplace128(dev):
    d, i, p, (rows, cols) = G.laplace3d(128, np.float64, jitter_seed=0)
    assert rows == 2097152 and d.shape[0] == 14581760
    D, I, P = to_dev(dev, d, i, p)
    A = sp.SparseCSRTensor((D, I, P), (rows, cols), clone=False)
    A.requires_grad = True
    C = A @ A
    assert C.nnz == 51742208
    Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(rows, cols, d, i, p, rows, cols, d, i, p)
    assert_same(host(C.indptr), Cp_ref, "C_indptr")
    assert_same(host(C.indices), Ci_ref, "C_indices")
    assert_same(host(C.data), Cd_ref, "C_data")
    gC = randn(1, C.nnz, np.float64)
    C.data.backward(to_dev(dev, gC)[0])
    gA_ref, gB_ref = oracle.spgemm_backward(gC, Ci_ref, Cp_ref, rows, cols, d, i, p, rows, cols, d, i, p)
    # both gradients are summed in the serial order on the plan; autograd adds the two
    assert_same(host(A.data.grad), gA_ref + gB_ref, "grad wrt A.values (grad_A + grad_B)")
    # ... and separately, through the binding
    gA, gB = ext.spgemm_backward(to_dev(dev, gC)[0], C.indices, C.indptr, rows, cols, D, I, P, rows, cols, D, I, P)
    assert_same(host(gA), gA_ref, "grad_A")
    assert_same(host(gB), gB_ref, "grad_B")
    # the first product built the product plan (the tests run in "eager" mode): a second one is the
    # planned numeric kernel alone, on the plan's pattern tensors, and the gradients above were the
    # mapped kernels'; on copies of the pattern tensors the search-based kernels run instead
    Cd2, Ci2, Cp2 = ext.spgemm_forward(rows, cols, D, I, P, rows, cols, D, I, P)
    assert Ci2.data_ptr() == C.indices.data_ptr() and Cp2.data_ptr() == C.indptr.data_ptr()
    assert_same(host(Cd2), Cd_ref, "C_data on the product plan")
    gA, gB = ext.spgemm_backward(to_dev(dev, gC)[0], C.indices.clone(), C.indptr.clone(), rows, cols, D, I, P,
                                 rows, cols, D, I, P)
    assert_same(host(gA), gA_ref, "grad_A (search-based, on A's transposed plan)")
    assert_same(host(gB), gB_ref, "grad_B (search-based, on A's transposed plan)")
    _binding.set_backward_mode("atomic")      # the stateless kernels: grad_B by atomics, tolerance
    gA, gB = ext.spgemm_backward(to_dev(dev, gC)[0], C.indices, C.indptr, rows, cols, D, I, P, rows, cols, D, I, P)
    assert_same(host(gA), gA_ref, "grad_A (stateless)")
    assert_close(host(gB), gB_ref, "grad_B (stateless)")


def test_cfg5_sptrsv_fp64_tril_poisson1024(dev):
    from numml_amd._binding import ops
    ops.clear_plan_cache()
    d, i, p, (n, _) = G.poisson2d_lower(1024, np.float64, diag_seed=0)
    assert n == 1048576 and d.shape[0] == 3143680
    b, g = randn(1, n, np.float64), randn(2, n, np.float64)
    D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
    L = sp.SparseCSRTensor((D, I, P), (n, n), clone=False)
    L.requires_grad = True
    Bv.requires_grad_(True)
    x = L.solve_triangular(upper=False, unit=False, b=Bv)
    x.backward(Gv)
    x_ref = oracle.sptrsv_forward(n, n, d, i, p, True, False, b)
    gA_ref, gb_ref = oracle.sptrsv_backward(g, x_ref, n, n, d, i, p, True, False)
    assert_same(host(x), x_ref, "x")
    assert_same(host(Bv.grad), gb_ref, "grad_b")
    assert_same(host(L.data.grad), gA_ref, "grad_A")
    assert ops.sptrsv_schedule(n, I, P, True)[0] == 2047       # rows on one anti-diagonal share a level
    assert ops.plan_cache_size() == 1                          # ... and that was the plan the solve used
    # residual of the full-size solve
    r = sps.csr_matrix((d, i, p), shape=(n, n)) @ host(x) - b
    assert np.linalg.norm(r) <= 1e-12 * np.linalg.norm(b) * 10


# ---- the same matrices in the other value type ---------------------------------------
# Lane and LDS layouts depend on the width of a value; the small-case tests cover both widths
# but only a few workgroups, these run the full grids.

def test_cfg2_matrix_in_fp64(dev):
    d, i, p, (rows, cols) = G.poisson2d(2048, np.float64, jitter_seed=0)
    x, g = randn(1, cols, np.float64), randn(2, rows, np.float64)
    D, I, P, X, Gv = to_dev(dev, d, i, p, x, g)
    y = ext.spgemv_forward(rows, cols, D, I, P, X)
    gA, gx = ext.spgemv_backward(Gv, rows, cols, D, I, P, X)
    gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
    assert_same(host(y), oracle.spgemv_forward(rows, cols, d, i, p, x), "y")
    assert_same(host(gA), gA_ref, "grad_A")
    assert_same(host(gx), gx_ref, "grad_x")


def test_cfg3_matrix_in_fp64_narrow_operand(dev):
    rows = cols = 1_000_000
    n = 16
    d, i, p, _ = G.powerlaw(rows, cols, target_nnz=16_000_000, seed=0, dtype=np.float64)
    B, gC = randn(1, (cols, n), np.float64), randn(2, (rows, n), np.float64)
    D, I, P, Bd, Gd = to_dev(dev, d, i, p, B, gC)
    C = host(ext.spdmm_forward(rows, cols, D, I, P, Bd))
    gA, gB = (host(v) for v in ext.spdmm_backward(rows, cols, D, I, P, Bd, Gd))
    A = sps.csr_matrix((d, i, p), shape=(rows, cols))
    C_ref, gB_ref = A @ B, A.T.tocsr() @ gC
    for got, want, what in ((C, C_ref, "C"), (gB, gB_ref, "grad_B")):
        assert np.all(np.abs(got - want) <= 1e-12 * np.abs(want) + 1e-12 * np.abs(want).max()), what
    # grad_A[k] = <gC[row(k)], B[col(k)]> on a sample of entries
    k = np.random.default_rng(3).integers(0, d.shape[0], 200_000)
    r = np.searchsorted(p, k, side="right") - 1
    want = np.einsum("kn,kn->k", gC[r], B[i[k]])
    assert np.all(np.abs(gA[k] - want) <= 1e-12 * np.abs(want) + 1e-12 * np.abs(want).max()), "grad_A"


def test_cfg4_matrix_in_fp32(dev):
    d, i, p, (rows, cols) = G.laplace3d(128, np.float32, jitter_seed=0)
    D, I, P = to_dev(dev, d, i, p)
    Cd, Ci, Cp = ext.spgemm_forward(rows, cols, D, I, P, rows, cols, D, I, P)
    Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(rows, cols, d, i, p, rows, cols, d, i, p)
    assert_same(host(Cp), Cp_ref, "C_indptr")
    assert_same(host(Ci), Ci_ref, "C_indices")
    assert_same(host(Cd), Cd_ref, "C_data")
    gC = randn(1, Cd_ref.shape[0], np.float32)
    gA, gB = ext.spgemm_backward(to_dev(dev, gC)[0], Ci, Cp, rows, cols, D, I, P, rows, cols, D, I, P)
    gA_ref, gB_ref = oracle.spgemm_backward(gC, Ci_ref, Cp_ref, rows, cols, d, i, p, rows, cols, d, i, p)
    assert_same(host(gA), gA_ref, "grad_A")
    assert_same(host(gB), gB_ref, "grad_B")
    Cd2, Ci2, Cp2 = ext.spgemm_forward(rows, cols, D, I, P, rows, cols, D, I, P)
    assert Ci2.data_ptr() == Ci.data_ptr()
    assert_same(host(Cd2), Cd_ref, "C_data on the product plan")


def test_cfg4_pattern_times_its_square(dev):
    """A (A A) on a 64^3 grid: named rows of B of 25 entries, rows of C of 63 -- the four-octet product
    plan on a few thousand workgroups (the small cases cover a handful)."""
    d, i, p, (rows, cols) = G.laplace3d(64, np.float64, jitter_seed=3)
    D, I, P = to_dev(dev, d, i, p)
    Sd, Si, Sp = ext.spgemm_forward(rows, cols, D, I, P, rows, cols, D, I, P)
    sd, si, sp_ = host(Sd), host(Si), host(Sp)
    assert int(np.diff(sp_).max()) == 25
    Cd, Ci, Cp = ext.spgemm_forward(rows, cols, D, I, P, rows, cols, Sd, Si, Sp)
    Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(rows, cols, d, i, p, rows, cols, sd, si, sp_)
    assert int(np.diff(Cp_ref).max()) == 63
    assert_same(host(Cp), Cp_ref, "C_indptr")
    assert_same(host(Ci), Ci_ref, "C_indices")
    assert_same(host(Cd), Cd_ref, "C_data")
    # again: the planned numeric kernel alone, on the plan's pattern tensors
    Cd2, Ci2, Cp2 = ext.spgemm_forward(rows, cols, D, I, P, rows, cols, Sd, Si, Sp)
    assert Ci2.data_ptr() == Ci.data_ptr() and Cp2.data_ptr() == Cp.data_ptr()
    assert_same(host(Cd2), Cd_ref, "C_data on the product plan")
    gC = randn(4, Cd_ref.shape[0], np.float64)
    gA, gB = ext.spgemm_backward(to_dev(dev, gC)[0], Ci, Cp, rows, cols, D, I, P, rows, cols, Sd, Si, Sp)
    gA_ref, gB_ref = oracle.spgemm_backward(gC, Ci_ref, Cp_ref, rows, cols, d, i, p, rows, cols, sd, si, sp_)
    assert_same(host(gA), gA_ref, "grad_A")
    assert_same(host(gB), gB_ref, "grad_B")


def test_cfg5_matrix_in_fp32(dev):
    d, i, p, (n, _) = G.poisson2d_lower(1024, np.float32, diag_seed=0)
    b, g = randn(1, n, np.float32), randn(2, n, np.float32)
    D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
    x = ext.sptrsv_forward(n, n, D, I, P, True, False, Bv)
    gA, gb = ext.sptrsv_backward(Gv, x, n, n, D, I, P, True, False, Bv)
    x_ref = oracle.sptrsv_forward(n, n, d, i, p, True, False, b)
    gA_ref, gb_ref = oracle.sptrsv_backward(g, x_ref, n, n, d, i, p, True, False)
    assert_same(host(x), x_ref, "x")
    assert_same(host(gb), gb_ref, "grad_b")
    assert_same(host(gA), gA_ref, "grad_A")


def test_structure_ops_on_the_cfg2_matrix_in_fp64(dev):
    """Transpose, linear combination, row sums, diagonal and their backwards over the full grid."""
    d, i, p, (rows, cols) = G.poisson2d(2048, np.float64, jitter_seed=0)
    e, j, q, _ = G.poisson2d(2048, np.float64, jitter_seed=1)
    g = randn(3, rows, np.float64)
    D, I, P, E, J, Q, Gv = to_dev(dev, d, i, p, e, j, q, g)
    At = ext.csr_transpose_forward(rows, cols, D, I, P)
    for got, want, what in zip(At, oracle.csr_transpose(rows, cols, d, i, p), ("At_data", "At_indices", "At_indptr", "At_to_A")):
        assert_same(host(got), want, what)
    one, half = torch.tensor(1.0, dtype=torch.float64), torch.tensor(-0.5, dtype=torch.float64)
    S = ext.splincomb_forward(rows, cols, one, D, I, P, half, E, J, Q)
    S_ref = oracle.splincomb_forward(rows, cols, 1.0, d, i, p, -0.5, e, j, q)
    for got, want, what in zip(S, S_ref, ("C_data", "C_indices", "C_indptr")):
        assert_same(host(got), want, what)
    gS = randn(4, S_ref[0].shape[0], np.float64)
    gs = ext.splincomb_backward(rows, cols, one, D, I, P, half, E, J, Q, to_dev(dev, gS)[0], S[1], S[2])
    for got, want, what in zip(gs, oracle.splincomb_backward(rows, cols, 1.0, d, i, p, -0.5, e, j, q, gS, S_ref[1], S_ref[2]),
                               ("grad_A", "grad_B")):
        assert_same(host(got), want, what)
    A = sps.csr_matrix((d, i, p), shape=(rows, cols))
    assert_same(host(ext.csr_row_sum_forward(rows, cols, D, I, P)), oracle.csr_row_sum_forward(rows, cols, d, i, p), "row sums")
    assert_same(host(ext.csr_extract_diagonal_forward(rows, cols, D, I, P)), A.diagonal(), "diagonal")
    assert_same(host(ext.csr_row_sum_backward(Gv, rows, cols, D, I, P)), np.repeat(g, np.diff(p)), "row sums backward")
    want = np.where(i == np.repeat(np.arange(rows), np.diff(p)), np.repeat(g, np.diff(p)), 0.0)
    assert_same(host(ext.csr_extract_diagonal_backward(Gv, rows, cols, D, I, P)), want, "diagonal backward")
