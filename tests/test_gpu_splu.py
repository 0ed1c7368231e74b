"""Sparse LU without pivoting and the direct solve on top of it (splu, spsolve_backward and
the ``linalg.splu / splu_solve / spsolve`` surface) on a HIP device.

The pattern with fill is integer work and the factors are computed in the reference's
operation order, so both are compared bit for bit with the CPU oracle
(cpp/sparse_csr_cpu.cpp:777-1016).  The solves go through the triangular solve, which
accumulates in double: fp32 1e-5 / fp64 1e-12 relative, as for that solve.
"""
import numpy as np
import pytest
import scipy.sparse as sps
import scipy.sparse.linalg as spla
import torch

import numml_amd
import oracle
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as mirror
from numml_amd import sparse as sp
from numml_amd.sparse import linalg
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

NAMES = ("M_data", "M_indices", "M_indptr", "Mt_data", "Mt_indices", "Mt_indptr")


def _from_scipy(m, dtype):
    m = m.tocsr()
    m.sort_indices()
    return m.data.astype(dtype), m.indices.astype(np.int64), m.indptr.astype(np.int64), m.shape


def _cases(dtype):
    yield "one", (np.full(1, 3, dtype), np.zeros(1, np.int64), np.array([0, 1], np.int64), (1, 1))
    yield "diagonal", _from_scipy(sps.diags(np.arange(1, 8, dtype=np.float64)), dtype)
    yield "tridiag12", G.tridiag(12, dtype)
    yield "tridiag700", G.tridiag(700, dtype)
    yield "poisson6", G.poisson2d(6, dtype, 1)
    yield "poisson24", G.poisson2d(24, dtype, 1)
    yield "random40", _from_scipy(sps.random(40, 40, 0.08, random_state=3, dtype=np.float64) + sps.eye(40) * 4.0, dtype)
    a = sps.random(25, 25, 0.1, random_state=7, dtype=np.float64)
    yield "symmetric25", _from_scipy(a + a.T + sps.eye(25) * 6.0, dtype)
    # unsymmetric pattern, rows longer than a wavefront, an arrow that fills the matrix
    b = sps.random(300, 300, 0.02, random_state=11, dtype=np.float64) + sps.eye(300) * 9.0
    yield "random300", _from_scipy(b, dtype)
    arrow = sps.lil_matrix((90, 90))
    arrow.setdiag(5.0)
    arrow[0, :] = 1.0
    arrow[:, 0] = 1.0
    arrow[0, 0] = 90.0
    yield "arrow90", _from_scipy(arrow, dtype)
    # the arrow the other way round (dense LAST row and column) does not fill, but its last column has
    # more entries than a wavefront keeps in LDS and its last row more than a wavefront has lanes
    n = 1300
    back = sps.lil_matrix((n, n))
    back.setdiag(4.0 + np.arange(n) % 3)
    back[n - 1, :] = 0.5
    back[:, n - 1] = -0.25
    back[n - 1, n - 1] = 3.0 * n
    yield "back_arrow1300", _from_scipy(back, dtype)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("binding", ["compiled", "ctypes"])
def test_splu_matches_the_oracle_bit_for_bit(dev, dtype, binding):
    ext = numml_amd.load_compiled() if binding == "compiled" else mirror
    for name, (d, i, p, (n, _)) in _cases(dtype):
        print("case", name, dtype.__name__, binding, flush=True)
        out = ext.splu(n, n, *to_dev(dev, d, i, p))
        want = oracle.splu(n, n, d, i, p)
        for got, ref, what in zip(out, want, NAMES):
            assert_same(host(got), ref, f"{name} {what}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_spsolve_backward_matches_the_oracle(dev, dtype):
    ext = numml_amd.load_compiled()
    for name, (d, i, p, (n, _)) in _cases(dtype):
        print("case", name, dtype.__name__, flush=True)
        M = oracle.splu(n, n, d, i, p)
        gx, x = randn(1, n, dtype), randn(2, n, dtype)
        want = oracle.spsolve_backward(gx, x, n, n, M[3], M[4], M[5], d, i, p)
        got = ext.spsolve_backward(*to_dev(dev, gx, x), n, n, *to_dev(dev, M[3], M[4], M[5], d, i, p))
        assert_close(host(got[1]), want[1], f"{name} grad_b")
        assert_close(host(got[0]), want[0], f"{name} grad_A")


def test_poisson_factors_reproduce_the_matrix_and_solve(dev):
    # 64 x 64 grid in natural ordering: the band fills (about half a million entries)
    d, i, p, (n, _) = G.poisson2d(64, np.float64, 1)
    A = sp.SparseCSRTensor(tuple(to_dev(dev, d, i, p)), (n, n))
    LU = linalg.splu(A)
    want = oracle.splu(n, n, d, i, p)
    assert_same(host(LU.indptr), want[2], "M_indptr")
    assert_same(host(LU.indices), want[1], "M_indices")
    assert_same(host(LU.data), want[0], "M_data")
    M = sps.csr_matrix((host(LU.data), host(LU.indices), host(LU.indptr)), shape=(n, n))
    Lf = sps.tril(M, -1) + sps.eye(n)
    Uf = sps.triu(M)
    As = sps.csr_matrix((d, i, p), shape=(n, n))
    assert abs(Lf @ Uf - As).max() < 1e-11
    b = randn(3, n, np.float64)
    x = linalg.splu_solve(LU, to_dev(dev, b)[0])
    xs = spla.spsolve(As.tocsc(), b)
    assert np.allclose(host(x), xs, rtol=1e-9, atol=1e-9 * np.abs(xs).max())


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_spsolve_gradients_against_dense_autograd(dev, dtype):
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    tol = 2e-4 if dtype == np.float32 else 1e-10
    for name, (d, i, p, (n, _)) in _cases(dtype):
        if name in ("tridiag700", "back_arrow1300"):
            continue
        D, I, P = to_dev(dev, d, i, p)
        A = sp.SparseCSRTensor((D.clone(), I, P), (n, n))
        A.requires_grad = True
        b = to_dev(dev, randn(4, n, dtype))[0].requires_grad_(True)
        w = to_dev(dev, randn(5, n, dtype))[0]
        x = linalg.spsolve(A, b)
        (x * w).sum().backward()
        # dense check in double on the host
        Ad = torch.tensor(sps.csr_matrix((d, i, p), shape=(n, n)).toarray(), dtype=torch.float64, requires_grad=True)
        bd = torch.tensor(host(b.detach()), dtype=torch.float64, requires_grad=True)
        xd = torch.linalg.solve(Ad, bd)
        (xd * torch.tensor(host(w), dtype=torch.float64)).sum().backward()
        scale = float(xd.detach().abs().max())
        assert np.allclose(host(x.detach()), xd.detach().numpy(), rtol=tol, atol=tol * scale), name
        assert x.dtype == tdt
        assert np.allclose(host(b.grad), bd.grad.numpy(), rtol=tol, atol=tol * float(bd.grad.abs().max())), name
        rows = np.repeat(np.arange(n), np.diff(p))
        gA = Ad.grad.numpy()[rows, i]
        assert np.allclose(host(A.grad.data), gA, rtol=tol, atol=tol * float(np.abs(gA).max())), name


def test_errors(dev):
    d, i, p, _ = G.random_csr(5, 7, 0.5, 1, np.float64)
    with pytest.raises(RuntimeError, match="square"):
        numml_amd.load_compiled().splu(5, 7, *to_dev(dev, d, i, p))
    with pytest.raises(RuntimeError, match="square"):
        mirror.splu(5, 7, *to_dev(dev, d, i, p))
    with pytest.raises(RuntimeError, match="HIP devices only"):
        mirror.splu(5, 5, torch.ones(5), torch.arange(5), torch.arange(6))


def test_pattern_is_computed_once_per_structure(dev):
    d, i, p, (n, _) = G.poisson2d(12, np.float64, 1)
    D, I, P = to_dev(dev, d, i, p)
    for ext in (numml_amd.load_compiled(), mirror):
        ext.clear_plan_cache()
        a = ext.splu(n, n, D, I, P)
        b = ext.splu(n, n, D * 2.0, I, P)
        for k in (1, 2, 4, 5):                       # the index tensors are shared between the calls
            assert a[k].data_ptr() == b[k].data_ptr()
        assert_same(host(b[0]), oracle.splu(n, n, d * 2.0, i, p)[0], "values follow the new data")
        a[1][0] = a[1][0]                            # an in-place edit invalidates the cached pattern
        c = ext.splu(n, n, D, I, P)
        assert c[1].data_ptr() != a[1].data_ptr()
        assert_same(host(c[0]), host(a[0]), "rebuilt")


def test_numeric_phase_gives_up_instead_of_waiting_forever(dev):
    # a poll limit of 1 on a matrix whose columns form one dependency chain: the kernel must
    # leave and the call report it (or, if every dependency happened to be ready, succeed)
    import ctypes
    from numml_amd import _lib
    L = _lib.lib()
    d, i, p, (n, _) = G.tridiag(700, np.float64)
    M = mirror.splu(n, n, *to_dev(dev, d, i, p))
    want = host(M[3])
    As = sps.csr_matrix((d, i, p), shape=(n, n)).T.tocsr()      # A^T on its own pattern: tridiagonal has no fill
    As.sort_indices()
    Td, Ti, Tp = to_dev(dev, As.data, As.indices.astype(np.int64), As.indptr.astype(np.int64))
    nbytes = ctypes.c_size_t(0)
    assert L.nm_splu_numeric_bytes(n, ctypes.byref(nbytes)) == 0
    work = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    rc = L.nm_splu_numeric(1, n, Td.data_ptr(), Ti.data_ptr(), Tp.data_ptr(), work.data_ptr(), nbytes.value, 1,
                           stream)
    if rc != 0:
        assert b"polls" in L.nm_last_error()
    else:
        assert_same(host(Td), want, "factors")
    # the device is fine afterwards
    Td2 = to_dev(dev, As.data)[0]
    assert L.nm_splu_numeric(1, n, Td2.data_ptr(), Ti.data_ptr(), Tp.data_ptr(), work.data_ptr(), nbytes.value, 0,
                             stream) == 0
    assert_same(host(Td2), want, "factors after the failed call")


def test_pattern_scratch_is_bounded(dev):
    # the pattern pass gives every wavefront 9 bytes of scratch per row; the number of wavefronts
    # is cut so that the total stays near 1 GiB (the walk itself costs O(rows) per row for a chain
    # like this one, as in the reference, so the size here is moderate)
    import ctypes
    from numml_amd import _lib
    nbytes = ctypes.c_size_t(0)
    assert _lib.lib().nm_splu_symbolic_bytes(400_000, ctypes.byref(nbytes)) == 0
    assert nbytes.value < 1.2 * 2 ** 30
    n = 30_000
    assert _lib.lib().nm_splu_symbolic_bytes(n, ctypes.byref(nbytes)) == 0
    assert nbytes.value < 1.2 * 2 ** 30       # 4096 wavefronts would need 1.1 GB: one step under the cut
    d, i, p, _ = G.tridiag(n, np.float64)
    print("case tridiag", n, flush=True)
    M = numml_amd.load_compiled().splu(n, n, *to_dev(dev, d, i, p))
    assert_same(host(M[1]), i, "no fill")
    assert_same(host(M[2]), p, "no fill")
    # u_0 = 2, l_k = -1 / u_{k-1}, u_k = 2 - l_k * (-1)
    u = np.empty(n)
    lo = np.empty(n)
    u[0] = 2.0
    for k in range(1, n):
        lo[k] = -1.0 / u[k - 1]
        u[k] = 2.0 - lo[k] * -1.0
    got = host(M[0])
    diag_pos = p[:-1] + (np.arange(n) > 0)
    assert np.array_equal(got[diag_pos], u)
    assert np.array_equal(got[p[1:-1]], lo[1:])
