"""The scenarios of the reference's own test-suite (numml/tests/test_spmv.py, test_spdmm.py,
test_spmm.py, test_sptrsv.py, test_transpose.py, test_add.py, test_misc.py), written against
this package's ``SparseCSRTensor`` on a HIP device.

The reference compares its CUDA path with its CPU path; there is no CPU path here, so the
device results are compared with dense float64 arithmetic on the host and, for gradients,
with the closed forms the reference's tests state or with centred finite differences.
"""
import numpy as np
import pytest
import torch

from numml_amd import sparse as sp

pytestmark = pytest.mark.gpu

A_N, AL_N = 16, 2048      # the large matrix spans several wavefronts (test_spmv.py:8-10)


def tridiag(n, dev, dtype=torch.float32):
    return (sp.eye(n, dtype=dtype, device=dev) * 2 - sp.eye(n, k=-1, dtype=dtype, device=dev)
            - sp.eye(n, k=1, dtype=dtype, device=dev))


def dense64(A):
    return torch.tensor(A.to_scipy_csr().toarray(), dtype=torch.float64)


def relerr(x, xhat):
    x, xhat = x.double().cpu().flatten(), xhat.double().cpu().flatten()
    return float(torch.linalg.norm(x - xhat) / torch.linalg.norm(x))


def random_sparse(rows, cols, sparsity, gen, tri=None, include_diag=True):
    """numml/tests/common.py:13-80: ceil(sparsity * rows * cols) draws of a position, N(0,1) values."""
    nnz = int(np.ceil(sparsity * rows * cols))
    A_d = torch.zeros((rows, cols))
    r, c = torch.randint(rows, (nnz,), generator=gen), torch.randint(cols, (nnz,), generator=gen)
    A_d[r, c] = torch.randn(nnz, generator=gen)
    if tri == "upper":
        A_d = torch.triu(A_d, 0 if include_diag else 1)
    elif tri == "lower":
        A_d = torch.tril(A_d, 0 if include_diag else -1)
    return A_d, sp.SparseCSRTensor(A_d)


def sp_fd(f, A, h=1e-3):
    """Centred differences over the stored entries (numml/utils.py:28-62)."""
    out = torch.empty_like(A.data)
    for i in range(A.nnz):
        d = A.data.detach().clone()
        d[i] += h
        up = float(f(sp.SparseCSRTensor((d, A.indices, A.indptr), A.shape)))
        d[i] -= 2 * h
        dn = float(f(sp.SparseCSRTensor((d, A.indices, A.indptr), A.shape)))
        out[i] = (up - dn) / (2 * h)
    return out


def reg_fd(f, x, h=1e-3):
    out = torch.empty_like(x)
    for i in range(x.numel()):
        d = x.detach().clone()
        d[i] += h
        up = float(f(d))
        d[i] -= 2 * h
        out[i] = (up - float(f(d))) / (2 * h)
    return out


# ------------------------------------------------------------------------------ test_spmv.py

def test_spmv_zeros_and_elementary(dev):
    A = tridiag(A_N, dev)
    assert torch.all((A @ torch.zeros(A_N, device=dev)) == 0)
    for i in range(A_N):
        e = torch.zeros(A_N, device=dev)
        e[i] = 1.
        Ae = A @ e                       # column i of A
        assert Ae[i] == 2
        if i > 0:
            assert Ae[i - 1] == -1
        if i < A_N - 1:
            assert Ae[i + 1] == -1


@pytest.mark.parametrize("n,tol", [(A_N, 1e-6), (AL_N, 1e-6)])
def test_spmv_random(dev, n, tol):
    A = tridiag(n, dev)
    A_d = dense64(A)
    gen = torch.Generator().manual_seed(n)
    for _ in range(20):
        b = torch.rand(n, generator=gen)
        assert relerr(A_d @ b.double(), A @ b.to(dev)) < tol


def test_spmv_backward(dev):
    AL = tridiag(AL_N, dev)
    gen = torch.Generator().manual_seed(3)
    rows = AL.row_indices.cpu()
    for _ in range(5):
        mult, x = torch.rand(AL_N, generator=gen), torch.rand(AL_N, generator=gen)
        Ag = AL.copy()
        Ag.requires_grad = True
        xg = x.to(dev).requires_grad_(True)
        ((Ag @ xg) * mult.to(dev)).sum().backward()
        # grad_A = outer(grad_w, x) on A's pattern, grad_x = A^T grad_w (A is symmetric)
        assert relerr(mult[rows] * x[AL.indices.cpu()], Ag.grad.data) < 1e-7
        assert relerr((AL @ mult.to(dev)), xg.grad) < 1e-7


# ----------------------------------------------------------------------------- test_spdmm.py

def test_spdmm_identity_and_random(dev):
    rng = np.random.default_rng(0)
    gen = torch.Generator().manual_seed(0)
    for _ in range(10):
        nr, nc = int(rng.integers(10, 1000)), int(rng.integers(5, 15))
        X = torch.randn(nr, nc, generator=gen).to(dev)
        assert torch.equal(X, sp.eye(nr, device=dev) @ X)
    for n in (A_N, AL_N):
        A = tridiag(n, dev)
        A_d = dense64(A)
        for _ in range(5):
            X = torch.randn(n, int(rng.integers(3, 10)), generator=gen)
            assert torch.allclose(A_d @ X.double(), (A @ X.to(dev)).cpu().double(), atol=1e-5)


def test_spdmm_backward(dev):
    AL, A = tridiag(AL_N, dev), tridiag(A_N, dev)
    gen = torch.Generator().manual_seed(1)
    rows, cols = AL.row_indices.cpu(), AL.indices.cpu()
    for nc in (3, 4, 6):
        X, gC = torch.randn(AL_N, nc, generator=gen), torch.randn(AL_N, nc, generator=gen)
        Ag = AL.copy()
        Ag.requires_grad = True
        ((Ag @ X.to(dev)) * gC.to(dev)).sum().backward()
        want = (gC[rows].double() * X[cols].double()).sum(1)          # gA_ij = sum_k gC_ik b_jk
        assert torch.allclose(Ag.grad.data.cpu().double(), want, atol=1e-5)
        Xs = torch.randn(A_N, nc, generator=gen).to(dev).requires_grad_(True)
        gCs = torch.randn(A_N, nc, generator=gen)
        ((A @ Xs) * gCs.to(dev)).sum().backward()
        assert torch.allclose(Xs.grad.cpu().double(), dense64(A).T @ gCs.double(), atol=1e-5)


# ------------------------------------------------------------------------------ test_spmm.py

def _interp(dev):
    P_d = torch.zeros((A_N, 4))
    for i in range(4):
        P_d[i * 4:(i + 1) * 4, i] = 1.
    return P_d, sp.SparseCSRTensor(P_d).to(dev)


def test_spspmm_matmat_and_skinny(dev):
    for n in (A_N, AL_N):
        A = tridiag(n, dev)
        B = (-A).copy()
        C = A @ B
        assert torch.allclose(dense64(A) @ dense64(B), dense64(C))
    A = tridiag(A_N, dev)
    P_d, P = _interp(dev)
    AH = P.T @ A @ P
    assert torch.allclose(dense64(AH), P_d.T.double() @ dense64(A) @ P_d.double())


def test_spspmm_gradients(dev):
    AL = tridiag(AL_N, dev)
    BL = (-AL).copy()
    mask = dense64(AL) != 0
    for wrt in ("A", "B"):
        Ag, Bg = AL.copy(), BL.copy()
        (Ag if wrt == "A" else Bg).requires_grad = True
        C = Ag @ Bg
        C.sum().backward()
        gC = torch.tensor(C.to_scipy_csr().toarray() != 0, dtype=torch.float64)   # ones on C's pattern
        if wrt == "A":      # (grad_C B^T) on mask(A)
            want, got = (gC @ dense64(BL).T) * mask, dense64(Ag.grad)
        else:               # (A^T grad_C) on mask(B)
            want, got = (dense64(AL).T @ gC) * mask, dense64(Bg.grad)
        assert torch.allclose(want, got)


def test_spspmm_skinny_gradients_against_finite_differences(dev):
    A = tridiag(A_N, dev)
    P_d, P = _interp(dev)
    Ag = A.copy()
    Ag.requires_grad = True
    (P.T @ Ag @ P).sum().backward()
    assert relerr(sp_fd(lambda M: (P.T @ M @ P).sum(), A), Ag.grad.data) < 1e-3
    Pg = P.copy()
    Pg.requires_grad = True
    (Pg.T @ A @ Pg).sum().backward()
    assert relerr(sp_fd(lambda M: (M.T @ A @ M).sum(), P), Pg.grad.data) < 1e-3


# ---------------------------------------------------------------------------- test_sptrsv.py

def test_sptrsv_identity(dev):
    N = 32
    I = sp.eye(N, device=dev)
    gen = torch.Generator().manual_seed(2)
    for _ in range(3):
        x = torch.randn(N, generator=gen).to(dev)
        for upper in (False, True):
            for unit in (False, True):
                assert torch.allclose(I.solve_triangular(upper, unit, x), x)


@pytest.mark.parametrize("upper", [False, True])
def test_sptrsv_bidiagonal(dev, upper):
    N, k = 32, (1 if upper else -1)
    gen = torch.Generator().manual_seed(4)
    A = sp.eye(N, device=dev) * 2 - sp.eye(N, k=k, device=dev)
    Au = sp.eye(N, device=dev) - sp.eye(N, k=k, device=dev) * 2
    for M, unit in ((A, False), (Au, True)):
        for _ in range(5):
            b = M @ torch.randn(N, generator=gen).to(dev)
            x = M.solve_triangular(upper, unit, b)
            assert float(torch.linalg.norm(b - M @ x) / torch.linalg.norm(b)) < 1e-5


def test_sptrsv_random_lower(dev):
    gen = torch.Generator().manual_seed(5)
    for _ in range(5):
        N = int(torch.randint(32, 2048, (1,), generator=gen))
        _, A = random_sparse(N, N, 0.05, gen, tri="lower", include_diag=False)
        A = (A.to(dev) + sp.eye(N, device=dev) * 2.).double()
        b = torch.randn(N, dtype=torch.double, generator=gen)
        x = A.solve_triangular(False, False, b.to(dev))
        want = torch.linalg.solve_triangular(dense64(A), b[:, None], upper=False)[:, 0]
        assert torch.allclose(x.cpu(), want, rtol=1e-8, atol=1e-8 * float(want.abs().max()))
        assert float(torch.linalg.norm(b.to(dev) - A @ x) / torch.linalg.norm(b)) < 1e-5


@pytest.mark.parametrize("upper", [False, True])
def test_sptrsv_gradients_against_finite_differences(dev, upper):
    N, k = 32, (1 if upper else -1)
    gen = torch.Generator().manual_seed(6)
    A = (sp.eye(N, device=dev) * 2 - sp.eye(N, k=k, device=dev)).double()
    Au = (sp.eye(N, device=dev) - sp.eye(N, k=k, device=dev) * 2).double()
    for M, unit in ((A, False), (Au, True)):
        b = (M @ torch.randn(N, dtype=torch.double, generator=gen).to(dev)).detach()
        Mg = M.copy()
        Mg.requires_grad = True
        bg = b.clone().requires_grad_(True)
        Mg.solve_triangular(upper, unit, bg).sum().backward()
        fd_b = reg_fd(lambda v: M.solve_triangular(upper, unit, v).sum(), b, h=1e-5)
        assert relerr(fd_b, bg.grad) < 1e-3
        if not unit:
            fd_A = sp_fd(lambda T: T.solve_triangular(upper, False, b).sum(), M, h=1e-5)
            assert relerr(fd_A, Mg.grad.data) < 1e-3
        else:
            # with a unit diagonal the stored diagonal is never read: its gradient is the closed form
            # -grad_b[i] x[i] all the same (cpp/sparse_csr_cpu.cpp:750-755), the rest matches differences
            off = (M.row_indices != M.indices).cpu()
            fd_A = sp_fd(lambda T: T.solve_triangular(upper, True, b).sum(), M, h=1e-5)
            assert relerr(fd_A[off], Mg.grad.data.cpu()[off]) < 1e-3


# ------------------------------------------------------------------------- test_transpose.py

def test_transpose_trivial(dev):
    A = tridiag(16, dev)
    At = A.T
    assert torch.equal(At.data, A.data) and torch.equal(At.indptr, A.indptr) and torch.equal(At.indices, A.indices)


@pytest.mark.parametrize("shape", [(512, 64), (64, 512)])
def test_transpose_random_and_gradient(dev, shape):
    gen = torch.Generator().manual_seed(shape[0])
    for _ in range(3):
        A_d, A = random_sparse(shape[0], shape[1], 0.5, gen)
        A = A.to(dev)
        assert torch.equal(A.T.to_dense().cpu(), A_d.T)
        A.requires_grad = True
        mult = torch.randn(A.nnz, generator=gen).to(dev)
        At = A.T
        At.data = At.data * mult
        At.sum().backward()
        # d/dA[r, c] of sum(A^T * W) = W[c, r]
        W = sp.SparseCSRTensor((mult, At.indices, At.indptr), At.shape).to_dense()
        assert torch.equal(A.grad.to_dense(), W.T * (A_d.to(dev) != 0))


# ------------------------------------------------------------------------------- test_add.py

def test_add_sub_random_and_gradient(dev):
    gen = torch.Generator().manual_seed(7)
    for _ in range(5):
        A_d, A = random_sparse(64, 64, 0.25, gen)
        B_d, B = random_sparse(64, 64, 0.25, gen)
        A, B = A.to(dev), B.to(dev)
        assert torch.equal((A + B).to_dense().cpu(), A_d + B_d)
        assert torch.equal((A - B).to_dense().cpu(), A_d - B_d)
    A_d, A = random_sparse(32, 32, 0.25, gen)
    B_d, B = random_sparse(32, 32, 0.25, gen)
    A, B = A.to(dev), B.to(dev)
    Ag, Bg = A.copy(), B.copy()
    Ag.requires_grad = True
    Bg.requires_grad = True
    (Ag + Bg).sum().backward()
    assert torch.equal(Ag.grad.data, torch.ones_like(A.data)) and torch.equal(Bg.grad.data, torch.ones_like(B.data))
    assert relerr(sp_fd(lambda M: (M + B).sum(), A, h=1e-2), Ag.grad.data) < 0.1
    assert relerr(sp_fd(lambda M: (A + M).sum(), B, h=1e-2), Bg.grad.data) < 0.1


# ------------------------------------------------------------------------------ test_misc.py

def test_to_dense_bands(dev):
    N = 16
    e = lambda k: sp.eye(N, k=k, device=dev)
    A_d = (e(0) * 3 + e(1) * 2 + e(-1) * 2 + e(2) + e(-2)).to_dense()
    for k, v in ((0, 3.), (1, 2.), (-1, 2.), (2, 1.), (-2, 1.), (3, 0.), (-3, 0.)):
        assert torch.all(torch.diag(A_d, k) == v)


# --------------------------------------------------------------- the rest of the container

def test_container_helpers(dev):
    x = torch.tensor([0., 2., 0., 3.], device=dev)
    y = torch.tensor([1., 0., 4.], device=dev)
    O = sp.spouter(x, y)                                       # numml/sparse/_csr.py:511-538
    assert torch.equal(O.to_dense(), torch.outer(x, y)) and O.nnz == 4
    A = tridiag(8, dev)
    d, i, p, shape = sp.unpack_csr(A)
    R = sp.repack_csr(d, i, p, shape)
    assert R.data.data_ptr() == A.data.data_ptr() and R.shape == A.shape
    coo = A.to_coo()
    assert coo.layout == torch.sparse_coo and torch.equal(coo.to_dense(), A.to_dense())
    assert np.array_equal(A.tocoo().toarray(), A.tocsr().toarray())
    assert torch.equal(A.conj().data, A.data) and torch.equal(abs(-A).data, A.abs().data)
    assert torch.equal((3 * A).data, (A * 3).data)
