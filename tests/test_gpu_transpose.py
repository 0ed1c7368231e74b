"""The explicit CSR transpose (csr_transpose_forward / _backward) on a HIP device.

Integer and copy work only, so everything is compared bit for bit with the CPU
oracle (cpp/sparse_csr_cpu.cpp:311-385), through both bindings, and through the
``SparseCSRTensor.T`` surface with gradients.
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


def _with_dense_columns(dtype):
    """30 000 rows; column 7 is stored in every row and column 400 in two rows of three (columns far
    longer than what the ordering kernel keeps in LDS, so their pieces are merged through memory),
    the rest random."""
    rows, cols = 30_000, 900
    rng = np.random.default_rng(11)
    r = np.concatenate([np.arange(rows), np.arange(rows)[np.arange(rows) % 3 != 0],
                        rng.integers(0, rows, 40_000)])
    c = np.concatenate([np.full(rows, 7), np.full(int((np.arange(rows) % 3 != 0).sum()), 400),
                        rng.integers(0, cols, 40_000)])
    rc = np.unique(np.stack([r, c], 1), axis=0)            # sorted by row, then column; no duplicates
    indptr = np.zeros(rows + 1, np.int64)
    np.cumsum(np.bincount(rc[:, 0], minlength=rows), out=indptr[1:])
    data = rng.standard_normal(rc.shape[0]).astype(dtype)
    return data, rc[:, 1].astype(np.int64), indptr, (rows, cols)


def _arrowhead(dtype, n=200_003):
    """Diagonal, dense first row, dense first column: one column of n entries (some fifty pieces of
    LDS keys and six merge passes in the ordering kernel, by a workgroup of its own)."""
    r = np.concatenate([np.arange(n), np.zeros(n - 1, np.int64), np.arange(1, n)])
    c = np.concatenate([np.arange(n), np.arange(1, n), np.zeros(n - 1, np.int64)])
    order = np.lexsort((c, r))
    r, c = r[order], c[order]
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(r, minlength=n), out=indptr[1:])
    data = np.random.default_rng(12).standard_normal(r.shape[0]).astype(dtype)
    return data, c.astype(np.int64), indptr, (n, n)


def _with_duplicates(dtype):
    """Stored entries with equal coordinates (the container keeps them, numml/sparse/_csr.py:78-99):
    the transpose must keep their storage order."""
    indptr = np.array([0, 3, 3, 7, 9], np.int64)
    indices = np.array([1, 1, 4, 0, 2, 2, 2, 1, 1], np.int64)
    data = np.arange(1, 10).astype(dtype)
    return data, indices, indptr, (4, 5)


def _cases(dtype):
    yield "tridiag16", G.tridiag(16, dtype)
    yield "poisson40", G.poisson2d(40, dtype, 1)
    yield "rect_wide", G.random_csr(37, 211, 0.08, 1, dtype)
    yield "rect_tall", G.random_csr(300, 19, 0.2, 2, dtype)
    yield "empty_rows_cols", G.random_csr(120, 130, 0.01, 3, dtype)
    yield "powerlaw", G.powerlaw(3000, 2500, 40000, max_deg=1200, seed=4, dtype=dtype)
    yield "dense_columns", _with_dense_columns(dtype)
    yield "arrowhead", _arrowhead(dtype)
    yield "duplicates", _with_duplicates(dtype)
    yield "no_entries", (np.zeros(0, dtype), np.zeros(0, np.int64), np.zeros(6, np.int64), (5, 7))
    yield "one", (np.ones(1, dtype), np.zeros(1, np.int64), np.array([0, 1], np.int64), (1, 1))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("binding", ["compiled", "ctypes"])
def test_transpose_forward_backward(dev, dtype, binding):
    ext = numml_amd.load_compiled() if binding == "compiled" else mirror
    for name, (d, i, p, (rows, cols)) in _cases(dtype):
        D, I, P = to_dev(dev, d, i, p)
        out = ext.csr_transpose_forward(rows, cols, D, I, P)
        ref = oracle.csr_transpose(rows, cols, d, i, p)
        for got, want, what in zip(out, ref, ("At_data", "At_indices", "At_indptr", "At_to_A_idx")):
            assert_same(host(got), want, f"{name} {what}")
        g = randn(5, d.shape[0], dtype)
        gA = ext.csr_transpose_backward(to_dev(dev, g)[0], out[3])
        assert_same(host(gA), oracle.csr_transpose_backward(g, ref[3]), f"{name} grad_A")
        # transposing twice gives the matrix back
        back = ext.csr_transpose_forward(cols, rows, out[0], out[1], out[2])
        assert_same(host(back[0]), d, f"{name} (A^T)^T data")
        assert_same(host(back[1]), i, f"{name} (A^T)^T indices")
        assert_same(host(back[2]), p, f"{name} (A^T)^T indptr")


def test_T_property_and_gradients(dev):
    d, i, p, (rows, cols) = G.random_csr(90, 70, 0.1, 7, np.float64)
    A = sp.SparseCSRTensor(tuple(to_dev(dev, d, i, p)), (rows, cols))
    A.requires_grad = True
    At = A.T
    assert At.shape == (cols, rows)
    assert torch.equal(At.to_dense(), A.to_dense().T)
    # y = A^T g: d(sum(w * y))/dA[k] = g[row(k)] * w[col(k)], the SpMV gradient with the roles swapped
    g, w = randn(1, rows, np.float64), randn(2, cols, np.float64)
    y = At @ to_dev(dev, g)[0]
    y.backward(to_dev(dev, w)[0])
    gA_ref, y_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, w)      # (g (x) w on the mask, A^T g)
    assert_close(host(y), y_ref, "A^T g")
    assert_same(host(A.data.grad), gA_ref, "gradient through the transpose")


def test_galerkin_triple_product_with_T(dev):
    # P^T A P with P^T taken by the transpose op (numml/tests/test_spmm.py:39-52)
    n, nc = 64, 16
    ad, ai, ap, _ = G.tridiag(n, np.float64)
    A = sp.SparseCSRTensor(tuple(to_dev(dev, ad, ai, ap)), (n, n))
    A.requires_grad = True
    r = np.arange(n)
    P = sp.SparseCSRTensor((torch.ones(n, dtype=torch.float64), (torch.from_numpy(r), torch.from_numpy(r // 4))),
                           shape=(n, nc)).to(dev)
    AH = P.T @ (A @ P)
    dense = P.to_dense().T @ A.to_dense().detach() @ P.to_dense()
    assert torch.allclose(AH.to_dense(), dense, atol=1e-12)
    AH.data.sum().backward()
    assert torch.allclose(A.data.grad, torch.ones_like(A.data))           # (P 1)(P 1)^T = 1 on A's pattern


def test_eye_and_diag_constructors(dev):
    for k in (-3, 0, 2):
        E = sp.eye(9, k=k, dtype=torch.float64, device=dev)
        assert torch.equal(E.to_dense(), torch.eye(9, dtype=torch.float64, device=dev).roll(k, 1).triu(k) if k >= 0
                           else torch.diag(torch.ones(9 + k, dtype=torch.float64, device=dev), k))
        x = torch.arange(1.0, 8.0, dtype=torch.float64, device=dev).requires_grad_(True)
        Dk = sp.diag(x, k=k)
        assert torch.equal(Dk.to_dense().detach(), torch.diag(x.detach(), k))
        (Dk @ torch.ones(Dk.shape[1], dtype=torch.float64, device=dev)).sum().backward()
        assert torch.equal(x.grad, torch.ones_like(x))
    with pytest.raises(RuntimeError, match="bandwidth"):
        sp.eye(4, k=4)
