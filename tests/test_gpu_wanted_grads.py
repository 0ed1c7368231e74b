"""A backward pass computes only the gradients somebody asked for, as the reference's GPU path
does (cpp/sparse_csr_cuda.cu:662, :682: `if (A_data.requires_grad())`, `if (B.requires_grad())`),
and forward passes run under ``torch.inference_mode()``.

The gradient that is computed alone must have the bits of the same gradient computed together
with the other one; the one that was not asked for comes back as ``None``.  Both bindings, both
value types, the stateless kernels and the kernels on cached plans.
"""
import numpy as np
import pytest
import torch

import oracle
from numml_amd import _binding
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as mirror
from numml_amd import sparse as sp
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

BINDINGS = [pytest.param(_binding.ops, id=_binding.name)]
if _binding.name != "ctypes":
    BINDINGS.append(pytest.param(mirror, id="ctypes"))


def _set_mode(ext, mode):
    if ext is mirror:
        mirror.BACKWARD_MODE = mode
    else:
        ext.set_backward_mode(mode)


def _get_mode(ext):
    return mirror.BACKWARD_MODE if ext is mirror else ext.backward_mode()


@pytest.fixture(params=["eager", "atomic"])
def mode(request):
    return request.param


def _flagged(t, flag):
    t = t.detach().clone()
    t.requires_grad_(flag)
    return t


def _check_pair(both, first_only, second_only, exact_first, exact_second, what):
    """both = [g1, g2] with no operand requiring a gradient; *_only = the calls in which one
    operand requires one."""
    assert both[0] is not None and both[1] is not None, f"{what}: a direct call gives both gradients"
    assert first_only[1] is None and second_only[0] is None, f"{what}: the gradient nobody asked for is None"
    (assert_same if exact_first else assert_close)(host(first_only[0]), host(both[0]), f"{what}: first gradient alone")
    (assert_same if exact_second else assert_close)(host(second_only[1]), host(both[1]), f"{what}: second gradient alone")


@pytest.mark.parametrize("ext", BINDINGS)
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_each_backward_computes_what_is_required(dev, ext, dtype, mode):
    old = _get_mode(ext)
    _set_mode(ext, mode)
    exact = mode == "eager"          # atomically summed gradients differ by rounding from run to run
    try:
        # SpMV
        d, i, p, (rows, cols) = G.poisson2d(48, dtype, jitter_seed=1)
        D, I, P, X, Gv = to_dev(dev, d, i, p, randn(1, cols, dtype), randn(2, rows, dtype))
        call = lambda a, x: ext.spgemv_backward(Gv, rows, cols, a, I, P, x)
        _check_pair(call(D, X), call(_flagged(D, True), X), call(D, _flagged(X, True)), True, exact, "spgemv")
        gA_ref, gx_ref = oracle.spgemv_backward(host(Gv), rows, cols, d, i, p, host(X))
        assert_same(host(call(_flagged(D, True), X)[0]), gA_ref, "spgemv grad_A alone vs oracle")
        assert_close(host(call(D, _flagged(X, True))[1]), gx_ref, "spgemv grad_x alone vs oracle")
        # SpMM, wide and narrow dense operands
        d, i, p, (rows, cols) = G.powerlaw(3000, 2500, 40000, max_deg=700, seed=3, dtype=dtype)
        for n in (64, 7):
            D, I, P, B, Gc = to_dev(dev, d, i, p, randn(4, (cols, n), dtype), randn(5, (rows, n), dtype))
            call = lambda a, b: ext.spdmm_backward(rows, cols, a, I, P, b, Gc)
            # (the dot products of long rows are folded differently by the fused and the row-major kernels)
            _check_pair(call(D, B), call(_flagged(D, True), B), call(D, _flagged(B, True)), False, exact, f"spdmm n={n}")
            gA_ref, gB_ref = oracle.spdmm_backward(rows, cols, d, i, p, host(B), host(Gc))
            assert_close(host(call(_flagged(D, True), B)[0]), gA_ref, "spdmm grad_A alone vs oracle")
            assert_close(host(call(D, _flagged(B, True))[1]), gB_ref, "spdmm grad_B alone vs oracle")
        # SpGEMM (two different operands)
        d, i, p, (rows, cols) = G.laplace3d(10, dtype, jitter_seed=2)
        e = G.laplace3d(10, dtype, jitter_seed=5)[0]
        D, I, P, E = to_dev(dev, d, i, p, e)
        Cd, Ci, Cp = ext.spgemm_forward(rows, cols, D, I, P, rows, cols, E, I, P)
        gC = to_dev(dev, randn(6, Cd.shape[0], dtype))[0]
        call = lambda a, b: ext.spgemm_backward(gC, Ci, Cp, rows, cols, a, I, P, rows, cols, b, I, P)
        _check_pair(call(D, E), call(_flagged(D, True), E), call(D, _flagged(E, True)), True, exact, "spgemm")
        gA_ref, gB_ref = oracle.spgemm_backward(host(gC), host(Ci), host(Cp), rows, cols, d, i, p, rows, cols, e, i, p)
        assert_same(host(call(_flagged(D, True), E)[0]), gA_ref, "spgemm grad_A alone vs oracle")
        assert_close(host(call(D, _flagged(E, True))[1]), gB_ref, "spgemm grad_B alone vs oracle")
        # SpTRSV
        d, i, p, (n, _) = G.poisson2d_lower(40, dtype, diag_seed=0)
        D, I, P, Bv, Gv = to_dev(dev, d, i, p, randn(7, n, dtype), randn(8, n, dtype))
        x = ext.sptrsv_forward(n, n, D, I, P, True, False, Bv)
        call = lambda a, b: ext.sptrsv_backward(Gv, x, n, n, a, I, P, True, False, b)
        _check_pair(call(D, Bv), call(_flagged(D, True), Bv), call(D, _flagged(Bv, True)), True, True, "sptrsv")
    finally:
        _set_mode(ext, old)


def test_autograd_leaves_the_unrequested_gradient_out(dev):
    """Through the container: a fixed operator with a trainable vector / dense operand (the
    reference's Krylov and GNN uses, numml/krylov.py:45, numml/nn.py:60) and the reverse."""
    dtype = np.float64
    d, i, p, (rows, cols) = G.poisson2d(32, dtype, jitter_seed=4)
    x, g = randn(1, cols, dtype), randn(2, rows, dtype)
    gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
    D, I, P, X, Gv = to_dev(dev, d, i, p, x, g)
    A = sp.SparseCSRTensor((D, I, P), (rows, cols))
    Xr = X.clone().requires_grad_(True)
    (A @ Xr).backward(Gv)                       # A fixed
    assert A.data.grad is None
    assert_same(host(Xr.grad), gx_ref, "grad_x with a fixed matrix")
    A.requires_grad = True
    (A @ X).backward(Gv)                        # x fixed
    assert X.grad is None
    assert_same(host(A.data.grad), gA_ref, "grad_A with a fixed vector")
    # SpMM with a fixed adjacency
    n = 48
    B, gC = randn(3, (cols, n), dtype), randn(4, (rows, n), dtype)
    Bd, Gc = to_dev(dev, B, gC)
    A2 = sp.SparseCSRTensor((D, I, P), (rows, cols))
    Br = Bd.clone().requires_grad_(True)
    (A2 @ Br).backward(Gc)
    assert A2.data.grad is None
    assert_same(host(Br.grad), oracle.spdmm_backward(rows, cols, d, i, p, B, gC)[1], "grad_B with a fixed matrix")
    # triangular solve with a fixed matrix
    d, i, p, (m, _) = G.poisson2d_lower(24, dtype, diag_seed=1)
    b, g = randn(5, m, dtype), randn(6, m, dtype)
    D, I, P, Bv, Gv = to_dev(dev, d, i, p, b, g)
    L = sp.SparseCSRTensor((D, I, P), (m, m))
    Br = Bv.clone().requires_grad_(True)
    L.solve_triangular(upper=False, unit=False, b=Br).backward(Gv)
    x_ref = oracle.sptrsv_forward(m, m, d, i, p, True, False, b)
    assert L.data.grad is None
    assert_same(host(Br.grad), oracle.sptrsv_backward(g, x_ref, m, m, d, i, p, True, False)[1], "grad_b, fixed matrix")


@pytest.mark.parametrize("mode", ["planned", "eager"])
def test_forward_passes_under_inference_mode(dev, mode):
    """Inference tensors carry no version counter; the plan bookkeeping must not ask for one.
    Every forward twice (the second call is the one that finds or builds plans), on operands
    made inside and outside the block."""
    ext = _binding.ops
    old = _binding.backward_mode()
    _binding.set_backward_mode(mode)
    dtype = np.float64
    try:
        d, i, p, (rows, cols) = G.laplace3d(8, dtype, jitter_seed=1)
        x = randn(1, cols, dtype)
        outside = to_dev(dev, d, i, p)
        ext.clear_plan_cache()
        with torch.inference_mode():
            inside = to_dev(dev, d, i, p)
            X = to_dev(dev, x)[0]
            for D, I, P in (outside, inside):
                A = sp.SparseCSRTensor((D, I, P), (rows, cols), clone=False)
                for _ in range(2):
                    y = A @ X
                    C = A @ A
                    E = C @ A                   # structure made inside the block
                    S = A + C
                    S2 = A - C
                assert_same(host(y), oracle.spgemv_forward(rows, cols, d, i, p, x), "y")
                Cd, Ci, Cp = oracle.spgemm_forward(rows, cols, d, i, p, rows, cols, d, i, p)
                assert_same(host(C.indices), Ci, "C_indices")
                assert_same(host(C.data), Cd, "C_data")
                Ed, Ei, Ep = oracle.spgemm_forward(rows, cols, Cd, Ci, Cp, rows, cols, d, i, p)
                assert_same(host(E.indptr), Ep, "E_indptr")
                assert_same(host(E.data), Ed, "E_data")
                Sd = oracle.splincomb_forward(rows, cols, 1.0, d, i, p, 1.0, Cd, Ci, Cp)[0]
                assert_same(host(S.data), Sd, "A + C")
            ld, li, lp, (m, _) = G.poisson2d_lower(20, dtype, diag_seed=2)
            b = randn(2, m, dtype)
            LD, LI, LP, Bv = to_dev(dev, ld, li, lp, b)
            L = sp.SparseCSRTensor((LD, LI, LP), (m, m), clone=False)
            for _ in range(2):
                xs = L.solve_triangular(upper=False, unit=False, b=Bv)
            assert_same(host(xs), oracle.sptrsv_forward(m, m, ld, li, lp, True, False, b), "x")
    finally:
        _binding.set_backward_mode(old)
