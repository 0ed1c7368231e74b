"""SpMV on a transposed-structure plan, through the C ABI: the packed structure of banded
patterns (one word per entry in the backward, 16-bit column offsets in the forward), patterns
whose offsets do not fit it, and both ways of addressing (32-bit offsets for arrays below
4 GiB, 64-bit ones beyond, forced here on small inputs).  Against the serial loops of
cpp/sparse_csr_cpu.cpp:29-35 and :60-73.
"""
import ctypes

import numpy as np
import pytest
import scipy.sparse as sps
import torch

import oracle
from numml_amd import _lib
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as ext
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]


def _csr(M, dtype):
    M = sps.csr_matrix(M).astype(dtype)
    M.sort_indices()
    return M.data.copy(), M.indices.astype(np.int64), M.indptr.astype(np.int64), M.shape


def _symmetric_band(n, offsets, seed, dtype):
    rng = np.random.default_rng(seed)
    diags = [rng.uniform(0.5, 1.5, n - abs(o)) for o in offsets]
    return _csr(sps.diags(diags, offsets, shape=(n, n)), dtype)


def _wide_rows(n, per_row, reach, seed, dtype):
    """Symmetric pattern, about 2 * per_row entries in every row within `reach` of the diagonal."""
    rng = np.random.default_rng(seed)
    r = np.repeat(np.arange(n), per_row)
    c = np.clip(r + rng.integers(-reach, reach + 1, r.size), 0, n - 1)
    M = sps.coo_matrix((np.ones(r.size), (r, c)), shape=(n, n)).tocsr()
    M = ((M + M.T) > 0).astype(np.float64)
    M.data = rng.uniform(0.5, 1.5, M.nnz)
    return _csr(M, dtype)


def _cross(n, seed, dtype):
    """A band plus one full row and one full column: a column (and a row) longer than a tile."""
    rng = np.random.default_rng(seed)
    M = sps.diags([np.ones(n - 1), np.ones(n), np.ones(n - 1)], [-1, 0, 1], shape=(n, n)).tolil()
    M[n // 3, :] = 1.0
    M[:, n // 3] = 1.0
    M = M.tocsr()
    M.data = rng.uniform(0.5, 1.5, M.nnz)
    return _csr(M, dtype)


def _cases(dtype):
    # name, matrix, (backward packed, forward packed), sums in storage order throughout
    yield "poisson64", G.poisson2d(64, dtype, jitter_seed=3), (1, 1), True
    yield "tridiag5000", G.tridiag(5000, dtype), (1, 1), True
    # an entry 40 000 columns from the diagonal: no 16-bit offset holds it
    yield "far_band", _symmetric_band(50000, [-40000, -1, 0, 1, 40000], 4, dtype), (0, 0), True
    # near the diagonal, but a row's mirror entries lie more than 32 767 positions away
    yield "thick_band", _wide_rows(3000, 20, 1500, 5, dtype), (0, 1), False
    # 3D seven-point pattern on 72^3: a column's entries one grid plane away lie 36 000 positions
    # from their mirror entries -- beyond the 16 bits of a plain packed word, inside the field a
    # block WITH a staging list has for the distance; every block of columns has a list
    yield "stencil3d_72", G.laplace3d(72, dtype, jitter_seed=7), (1, 1), True
    # the same followed by a tridiagonal block (three entries a column: no list, plain packed
    # words): both layouts of the word in one plan
    d3, i3, p3, (n3, _) = G.laplace3d(72, dtype, jitter_seed=8)
    dt_, it_, pt_, (nt_, _) = G.tridiag(5000, dtype)
    yield "stencil3d_then_tridiag", _csr(sps.block_diag([sps.csr_matrix((d3, i3, p3), shape=(n3, n3)),
                                                         sps.csr_matrix((dt_, it_, pt_), shape=(nt_, nt_))]),
                                         dtype), (1, 1), True
    # 4, 6 and 8 entries a column: blocks of 256 columns with exactly 1024, 1536 and 2048 entries,
    # i.e. the backward's tile with a list and no, two and four rounds behind its quads
    for per in (4, 6, 8):
        offs = [o for o in range(-per // 2, per // 2 + 1) if o != 0]
        yield f"band{per}", _symmetric_band(6000, offs, 10 + per, dtype), (1, 1), True
    yield "rectangular", G.random_csr(700, 300, 0.02, 5, dtype), (1, 1), True
    yield "cross", _cross(6000, 6, dtype), (1, 1), False
    # rows and columns of thousands of entries spread over 50 000 columns: the plain 32-bit arrays
    # on every path of the kernels (runs of columns, columns longer than a tile)
    yield "powerlaw50k", G.powerlaw(50000, 50000, target_nnz=400000, max_deg=6000, seed=9, dtype=dtype), (0, 0), False
    yield "powerlaw50k_T", _csr(sps.csr_matrix(G.powerlaw(50000, 50000, target_nnz=400000, max_deg=6000, seed=10,
                                                          dtype=dtype)[:3], shape=(50000, 50000)).T, dtype), (0, 0), False
    yield "empty", (np.zeros(0, dtype), np.zeros(0, np.int64), np.zeros(6, np.int64), (5, 4)), None, True


def _plan_flags(plan, rows, cols, nnz):
    a = lambda v: (v + 255) & ~255
    off = a((cols + 1) * 4) + 2 * a((nnz + 1) * 4) + a(((nnz + 63) // 64 + 1) * 4)
    return plan.mem[off:off + 12].cpu().view(torch.int32).tolist()


@pytest.mark.parametrize("dtype", DTYPES)
def test_planned_spmv_packed_and_plain_structure(dev, dtype):
    L = _lib.lib()
    dt = 0 if dtype == np.float32 else 1
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    try:
        for name, (d, i, p, (rows, cols)), packed, exact in _cases(dtype):
            nnz = d.shape[0]
            x, g = randn(1, cols, dtype), randn(2, rows, dtype)
            y_ref = oracle.spgemv_forward(rows, cols, d, i, p, x)
            gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
            D, I, P, X, Gd = to_dev(dev, d, i, p, x, g)
            plan = ext._TransposePlan(I, P, rows, cols, dev)
            if packed is not None:
                flags = _plan_flags(plan, rows, cols, nnz)
                assert (flags[1], flags[2]) == packed, f"{name}: plan flags {flags}"
            results = []
            for wide in (0, 1):
                assert L.nm_spgemv_configure(wide) == 0
                y = torch.full((rows,), 7.0, dtype=D.dtype, device=dev)
                gA = torch.full((nnz,), 7.0, dtype=D.dtype, device=dev)
                gx = torch.full((cols,), 7.0, dtype=D.dtype, device=dev)
                _lib.check(L.nm_spgemv_forward_planned(dt, rows, cols, nnz, ptr(D), ptr(plan.mem), ptr(X), ptr(y),
                                                       stream), "nm_spgemv_forward_planned")
                # the instantiation that takes blocks with a staging list through LDS: the same bits
                y_l = torch.full((rows,), 7.0, dtype=D.dtype, device=dev)
                _lib.check(L.nm_spgemv_forward_planned_lists(dt, rows, cols, nnz, ptr(D), ptr(plan.mem), ptr(X),
                                                             ptr(y_l), stream), "nm_spgemv_forward_planned_lists")
                # (rows that one lane sums in storage order -- fewer than 32 entries -- come out the
                # same bit for bit; a longer row is shared by a wavefront where its block does not fit
                # the tile, and the two builds have different tiles in fp64)
                if exact:
                    assert torch.equal(y, y_l), f"{name}: forward with and without staging lists"
                else:
                    assert_close(host(y_l), host(y), f"{name}: forward with and without staging lists")
                _lib.check(L.nm_spgemv_backward_planned(dt, rows, cols, nnz, ptr(D), ptr(plan.mem), ptr(X), ptr(Gd),
                                                        ptr(gA), ptr(gx), stream), "nm_spgemv_backward_planned")
                # the same for the backward: both builds, both gradients and each alone
                for gA_want, gx_want in ((True, True), (True, False), (False, True)):
                    gA_l = torch.full((nnz,), 7.0, dtype=D.dtype, device=dev) if gA_want else None
                    gx_l = torch.full((cols,), 7.0, dtype=D.dtype, device=dev) if gx_want else None
                    gA_p = torch.full((nnz,), 7.0, dtype=D.dtype, device=dev) if gA_want else None
                    gx_p = torch.full((cols,), 7.0, dtype=D.dtype, device=dev) if gx_want else None
                    _lib.check(L.nm_spgemv_backward_planned_lists(
                        dt, rows, cols, nnz, ptr(D), ptr(plan.mem), ptr(X), ptr(Gd),
                        ptr(gA_l) if gA_want else None, ptr(gx_l) if gx_want else None, stream),
                        "nm_spgemv_backward_planned_lists")
                    _lib.check(L.nm_spgemv_backward_planned(
                        dt, rows, cols, nnz, ptr(D), ptr(plan.mem), ptr(X), ptr(Gd),
                        ptr(gA_p) if gA_want else None, ptr(gx_p) if gx_want else None, stream),
                        "nm_spgemv_backward_planned")
                    if gA_want:
                        assert torch.equal(gA_l, gA_p), f"{name}: grad_A with and without staging lists"
                    if gx_want:
                        assert torch.equal(gx_l, gx_p), f"{name}: grad_x with and without staging lists"
                same = assert_same if exact else assert_close
                same(host(y), y_ref, f"{name} y (wide={wide})")
                assert_same(host(gA), gA_ref, f"{name} grad_A (wide={wide})")
                same(host(gx), gx_ref, f"{name} grad_x (wide={wide})")
                # one gradient at a time: the walk that does not fuse the two
                gA1 = torch.full((nnz,), 7.0, dtype=D.dtype, device=dev)
                gx1 = torch.full((cols,), 7.0, dtype=D.dtype, device=dev)
                _lib.check(L.nm_spgemv_backward_planned(dt, rows, cols, nnz, ptr(D), ptr(plan.mem), ptr(X), ptr(Gd),
                                                        ptr(gA1), None, stream), "nm_spgemv_backward_planned")
                _lib.check(L.nm_spgemv_backward_planned(dt, rows, cols, nnz, ptr(D), ptr(plan.mem), ptr(X), ptr(Gd),
                                                        None, ptr(gx1), stream), "nm_spgemv_backward_planned")
                assert_same(host(gA1), host(gA), f"{name} grad_A alone (wide={wide})")
                assert_same(host(gx1), host(gx), f"{name} grad_x alone (wide={wide})")
                results.append((host(y), host(gA), host(gx)))
            for a, b, what in zip(results[0], results[1], ("y", "grad_A", "grad_x")):
                assert_same(a, b, f"{name} {what}: 32-bit against 64-bit offsets")
    finally:
        assert L.nm_spgemv_configure(0) == 0
