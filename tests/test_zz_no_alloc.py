"""nm_sptrsv_solve_static: the triangular solve whose scratch is the library's own
device array, for callers that cannot allocate.  Called through the C ABI and
compared bit for bit with nm_sptrsv_solve (caller-provided scratch) on two calls in
a row, the second on a smaller system, so that what the first call left in the
shared array is seen to do no harm; oversized systems are refused."""
import ctypes

import numpy as np
import pytest
import torch

from numml_amd import _lib, generators as G

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


class _Plan:
    def __init__(self, idx, ptr, rows, lower, dev):
        L = _lib.lib()
        nnz = idx.shape[0]
        pb, wb = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _lib.check(L.nm_sptrsv_plan_bytes(rows, nnz, ctypes.byref(pb), ctypes.byref(wb)), "plan_bytes")
        self.mem = torch.empty(max(pb.value, 8), dtype=torch.uint8, device=dev)
        work = torch.empty(max(wb.value, 8), dtype=torch.uint8, device=dev)
        self.handle = ctypes.c_void_p(0)
        _lib.check(L.nm_sptrsv_analyse(rows, nnz, _ptr(idx), _ptr(ptr), int(lower), _ptr(self.mem), pb.value,
                                       _ptr(work), wb.value, ctypes.byref(self.handle), None), "analyse")
        self.rows, self.nnz = rows, nnz

    def close(self):
        _lib.lib().nm_sptrsv_plan_destroy(self.handle)


def _both_ways(dev, n, np_dtype, transposed, unit, seed):
    """x from nm_sptrsv_solve and from nm_sptrsv_solve_static on tril(Poisson n x n)."""
    L = _lib.lib()
    d, i, p, (rows, _) = G.poisson2d_lower(n, np_dtype, diag_seed=seed)
    b = np.random.default_rng(seed + 1).standard_normal(rows).astype(np_dtype)
    D, I, P, B = (torch.from_numpy(a).to(dev) for a in (d, i, p, b))
    plan = _Plan(I, P, rows, True, dev)
    dt = _lib.NM_F32 if np_dtype == np.float32 else _lib.NM_F64
    nb = ctypes.c_size_t(0)
    _lib.check(L.nm_sptrsv_solve_bytes(rows, plan.nnz, ctypes.byref(nb)), "solve_bytes")
    work = torch.empty(nb.value, dtype=torch.uint8, device=dev)
    x_ref = torch.empty_like(B)
    _lib.check(L.nm_sptrsv_solve(plan.handle, dt, int(transposed), _ptr(D), int(unit), _ptr(B), _ptr(x_ref),
                                 _ptr(work), nb.value, None), "nm_sptrsv_solve")
    x = torch.full_like(B, float("nan"))
    _lib.check(L.nm_sptrsv_solve_static(plan.handle, dt, int(transposed), _ptr(D), int(unit), _ptr(B), _ptr(x),
                                        None), "nm_sptrsv_solve_static")
    torch.cuda.synchronize()
    out = x.cpu().numpy(), x_ref.cpu().numpy()
    plan.close()
    return out


def test_static_solve_equals_the_solve_with_caller_scratch_twice_in_a_row(dev):
    cap = ctypes.c_size_t(0)
    _lib.check(_lib.lib().nm_sptrsv_solve_static_capacity(ctypes.byref(cap)), "capacity")
    assert cap.value == 64 << 20
    # first a larger system, then a smaller one on the same (now dirty) built-in array
    for n, np_dtype, transposed, unit, seed in ((300, np.float64, False, False, 0),
                                                (97, np.float64, False, False, 3),
                                                (200, np.float32, True, False, 5),
                                                (33, np.float32, True, True, 7)):
        x, x_ref = _both_ways(dev, n, np_dtype, transposed, unit, seed)
        assert np.all(np.isfinite(x_ref))
        assert np.array_equal(x, x_ref), f"n={n} {np_dtype.__name__} transposed={transposed} unit={unit}"


def test_static_solve_refuses_what_does_not_fit(dev):
    L = _lib.lib()
    n = 1024     # 1 048 576 rows: needs about 134 MB of scratch
    d, i, p, (rows, _) = G.poisson2d_lower(n, np.float64, diag_seed=0)
    D, I, P = (torch.from_numpy(a).to(dev) for a in (d, i, p))
    B = torch.zeros(rows, dtype=torch.float64, device=dev)
    plan = _Plan(I, P, rows, True, dev)
    x = torch.empty_like(B)
    rc = L.nm_sptrsv_solve_static(plan.handle, _lib.NM_F64, 0, _ptr(D), 0, _ptr(B), _ptr(x), None)
    assert rc == 4 and b"built-in" in L.nm_last_error()      # NM_ERR_UNSUPPORTED, nothing launched
    torch.cuda.synchronize()
    plan.close()
