"""Drop-in behaviour of the Python surface on a HIP device: routing of ``@``,
shape conventions, gradient plumbing and the structure-plan cache."""
import numpy as np
import pytest
import torch

import oracle
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as ext
from numml_amd import sparse as sp
from numml_amd.sparse import linalg
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu


def _A(dev, csr, grad=False):
    d, i, p, shape = csr
    A = sp.SparseCSRTensor(tuple(to_dev(dev, d, i, p)), shape)
    A.requires_grad = grad
    return A


def test_matmul_routes_and_keeps_singleton_dims(dev):
    csr = G.tridiag(16, np.float32)
    A = _A(dev, csr)
    Ad = A.to_dense()
    torch.manual_seed(0)
    x = torch.rand(16, device=dev)
    assert torch.allclose(A @ x, Ad @ x, atol=1e-6)     # atol: 2x_i - x_(i-1) - x_(i+1) cancels
    assert (A @ x.reshape(16, 1)).shape == (16, 1)          # spmv squeezes and restores (numml/sparse/_csr.py:656-657)
    assert (A @ x.reshape(1, 16, 1)).shape == (1, 16, 1)
    assert torch.all((A @ torch.zeros(16, device=dev)) == 0)
    for j in range(16):                                      # numml/tests/test_spmv.py:21-39
        e = torch.zeros(16, device=dev)
        e[j] = 1
        assert torch.equal(A @ e, Ad[:, j])
    X = torch.rand(16, 5, device=dev)
    assert torch.allclose(A @ X, Ad @ X, atol=1e-6)
    X3 = torch.rand(3, 4, 16, 5, device=dev)                 # batched: one flattened SpMM (:717-732)
    assert torch.allclose(A @ X3, torch.matmul(Ad, X3), atol=1e-6)
    C = A @ (-A)                                             # numml/tests/test_spmm.py:23-36
    assert isinstance(C, sp.SparseCSRTensor) and C.shape == (16, 16)
    assert torch.allclose(C.to_dense(), Ad @ (-Ad), atol=1e-6)


def test_galerkin_product_and_gradients_through_two_spgemms(dev):
    # P^T A P with a piecewise-constant P (numml/tests/test_spmm.py:39-52), here with P^T given explicitly
    n, nc = 64, 16
    A = _A(dev, G.tridiag(n, np.float64), grad=True)
    rows = np.arange(n)
    P = sp.SparseCSRTensor((torch.ones(n, dtype=torch.float64), (torch.from_numpy(rows), torch.from_numpy(rows // 4))),
                           shape=(n, nc)).to(dev)
    Pt = sp.SparseCSRTensor((torch.ones(n, dtype=torch.float64), (torch.from_numpy(rows // 4), torch.from_numpy(rows))),
                            shape=(nc, n)).to(dev)
    AH = Pt @ (A @ P)
    dense = Pt.to_dense() @ A.to_dense().detach() @ P.to_dense()
    assert torch.allclose(AH.to_dense(), dense, atol=1e-12)
    AH.data.sum().backward()
    # d/dA_ij sum(P^T A P) = (P 1)(P 1)^T restricted to A's pattern = 1 on every stored entry
    assert torch.allclose(A.data.grad, torch.ones_like(A.data))


def test_spgemm_same_operand_accumulates_both_gradients(dev):
    csr = G.random_csr(40, 40, 0.1, 3, np.float64)
    d, i, p, (n, _) = csr
    A = _A(dev, csr, grad=True)
    C = A @ A
    gC = randn(4, C.nnz, np.float64)
    C.data.backward(to_dev(dev, gC)[0])
    Cd, Ci, Cp = oracle.spgemm_forward(n, n, d, i, p, n, n, d, i, p)
    gA, gB = oracle.spgemm_backward(gC, Ci, Cp, n, n, d, i, p, n, n, d, i, p)
    assert_close(host(A.data.grad), gA + gB, "grad_A + grad_B")


def test_finite_differences_of_the_solve(dev):
    # numml/tests/test_sptrsv.py:113-240 checks gradients against finite differences
    d, i, p, (n, _) = G.random_tri(30, 0.15, 8, True, np.float64)
    D, I, P = to_dev(dev, d, i, p)
    b = to_dev(dev, randn(1, n, np.float64))[0].requires_grad_(True)
    A = sp.SparseCSRTensor((D, I, P), (n, n))
    A.requires_grad = True
    w = to_dev(dev, randn(2, n, np.float64))[0]
    f = lambda dat, rhs: (linalg.sptrsv.apply((n, n), dat, A.indices, A.indptr, True, False, rhs) * w).sum()
    f(A.data, b).backward()
    h = 1e-6
    for k in (0, 5, len(d) - 1):
        e = torch.zeros_like(A.data)
        e[k] = h
        fd = (f(A.data.detach() + e, b.detach()) - f(A.data.detach() - e, b.detach())) / (2 * h)
        assert abs(fd.item() - A.data.grad[k].item()) <= 1e-5 * max(1.0, abs(fd.item()))
    e = torch.zeros_like(b)
    e[3] = h
    fd = (f(A.data.detach(), b.detach() + e) - f(A.data.detach(), b.detach() - e)) / (2 * h)
    assert abs(fd.item() - b.grad[3].item()) <= 1e-5 * max(1.0, abs(fd.item()))


def test_solve_triangular_upper_unit_and_missing_diagonal(dev):
    d, i, p, (n, _) = G.random_tri(60, 0.1, 9, False, np.float64, diag=False)   # strictly upper, no diagonal
    A = _A(dev, (d, i, p, (n, n)))
    b = randn(3, n, np.float64)
    x = A.solve_triangular(upper=True, unit=True, b=to_dev(dev, b)[0])
    assert_same(host(x), oracle.sptrsv_forward(n, n, d, i, p, False, True, b), "unit upper solve")
    x = A.solve_triangular(upper=True, unit=False, b=to_dev(dev, b)[0])        # division by the absent diagonal
    assert_same(host(x), oracle.sptrsv_forward(n, n, d, i, p, False, False, b), "missing diagonal -> inf/nan")


def test_plan_cache_hits_and_invalidation(dev):
    ext.clear_plan_cache()
    d, i, p, (n, _) = G.poisson2d_lower(20, np.float64)
    D, I, P = to_dev(dev, d, i, p)
    b = to_dev(dev, randn(1, n, np.float64))[0]
    ext.sptrsv_forward(n, n, D, I, P, True, False, b)
    ext.sptrsv_forward(n, n, D, I, P, True, False, b)
    assert len(ext._plans) == 1
    ext.sptrsv_backward(b, b, n, n, D, I, P, True, False, b)      # same plan serves the transposed solve
    assert len(ext._plans) == 1
    ext.spgemv_backward(b, n, n, D, I, P, b)                       # transposed-structure plan is separate
    assert len(ext._plans) == 2
    # an in-place edit of the structure must not reuse the stale schedule
    d2, i2, p2, _ = G.bidiag(n, np.float64)
    D2, I2, P2 = to_dev(dev, d2, i2, p2)
    I3 = I2.clone()
    x_a = ext.sptrsv_forward(n, n, D2, I3, P2, True, False, b)
    I3[1] = 1                                                      # (1,0) -> (1,1): row 1 loses its dependency
    x_b = ext.sptrsv_forward(n, n, D2, I3, P2, True, False, b)
    i3 = host(I3)
    assert_same(host(x_b), oracle.sptrsv_forward(n, n, d2, i3, p2, True, False, host(b)), "after edit")
    assert not torch.equal(x_a, x_b)


def test_dtype_and_device_errors_on_device(dev):
    d, i, p, (n, _) = G.tridiag(8, np.float32)
    D, I, P = to_dev(dev, d, i, p)
    x = torch.ones(n, device=dev)
    with pytest.raises(RuntimeError, match="Long"):
        ext.spgemv_forward(n, n, D, I.int(), P, x)
    with pytest.raises(RuntimeError, match="same device"):
        ext.spdmm_forward(n, n, D, I, P, torch.ones(n, 2))
    with pytest.raises(RuntimeError, match="float32 or float64"):
        ext.spgemv_forward(n, n, D.half(), I, P, x.half())


def test_conjugate_gradients_and_training_through_the_solver(dev):
    # what the reference's Krylov code does with these operators (numml/krylov.py:83-155): a CG
    # loop whose only matrix operation is A @ p, differentiated end to end -- here the stencil
    # values of a 2-D Poisson operator are trained so that five CG steps solve A x = b better
    import scipy.sparse.linalg as spla
    d, i, p, (n, _) = G.poisson2d(24, np.float64, jitter_seed=None)
    A = sp.SparseCSRTensor(tuple(to_dev(dev, d, i, p)), (n, n))
    b = to_dev(dev, randn(1, n, np.float64))[0]

    def cg(A, b, iters):
        x = torch.zeros_like(b)
        r = b - A @ x
        q = r.clone()
        rs = r @ r
        for _ in range(iters):
            Aq = A @ q
            alpha = rs / (q @ Aq)
            x = x + alpha * q
            r = r - alpha * Aq
            rs_new = r @ r
            q = r + (rs_new / rs) * q
            rs = rs_new
        return x

    x = cg(A, b, 200)
    want = spla.spsolve(A.to_scipy_csr().tocsc(), host(b))
    assert np.allclose(host(x), want, rtol=1e-8, atol=1e-8 * np.abs(want).max())
    # gradient of a loss through five CG steps with respect to the stored values, against
    # the same loop in dense float64 autograd on the host
    A.requires_grad = True
    loss = ((A @ cg(A, b, 5) - b) ** 2).sum()
    loss.backward()
    Ad = torch.tensor(A.to_scipy_csr().toarray(), dtype=torch.float64, requires_grad=True)
    bh = torch.tensor(host(b))
    ((Ad @ cg(Ad, bh, 5) - bh) ** 2).sum().backward()
    rows = np.repeat(np.arange(n), np.diff(p))
    gA = Ad.grad.numpy()[rows, i]
    assert np.allclose(host(A.grad.data), gA, rtol=1e-8, atol=1e-10 * np.abs(gA).max())


def test_stream_probe_and_longest_row_through_the_c_abi(dev):
    """The two helper entry points callers use beside the operators: the plain streaming kernel
    (copies the first write_bytes of what it reads, leaves the rest of the destination alone,
    refuses sizes that are not multiples of 16) and the longest row of a pattern."""
    import ctypes
    from numml_amd import _lib
    L = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    src = torch.arange(1 << 16, dtype=torch.float32, device=dev)
    dst = torch.full((1 << 16,), -1.0, device=dev)
    half = src.numel() * 4 // 2
    _lib.check(L.nm_stream_probe(ptr(src), src.numel() * 4, ptr(dst), half, stream), "nm_stream_probe")
    assert torch.equal(dst[:1 << 15], src[:1 << 15]) and bool((dst[1 << 15:] == -1).all())
    _lib.check(L.nm_stream_probe(ptr(src), src.numel() * 4, None, 0, stream), "nm_stream_probe (read only)")
    assert L.nm_stream_probe(ptr(src), 24, ptr(dst), 16, stream) != 0          # not a multiple of 16
    assert L.nm_stream_probe(ptr(src), 64, ptr(dst), 128, stream) != 0         # writes more than it reads
    for lens in ([3, 0, 7, 2], [0, 0, 0], [5], list(np.random.default_rng(3).integers(0, 900, 5000))):
        indptr = torch.tensor(np.concatenate([[0], np.cumsum(lens)]).astype(np.int64), device=dev)
        work = torch.empty(4096, dtype=torch.uint8, device=dev)
        longest = ctypes.c_int64(-1)
        _lib.check(L.nm_csr_longest_row(len(lens), ptr(indptr), ptr(work), work.numel(), None,
                                        ctypes.byref(longest), stream), "nm_csr_longest_row")
        assert longest.value == max(lens)
