"""Stand-in for the reference's extension module ``numml_torch_cpp``.

Exports the eight hot-path functions with the reference's names, positional
signatures and return conventions (cpp/sparse_csr.cpp:307-319 binds them;
cpp/sparse_csr.hpp:32-105 declares them), implemented on the HIP kernels of
libnumml_hip.so.  torch is used for device memory (outputs and scratch come
from its caching allocator) and for the current stream, nothing else.

Unlike the reference there is no CPU implementation behind these functions:
tensors that are not on a HIP device raise ``RuntimeError``.
"""
import atexit
import collections
import ctypes
import os
import threading

import torch

from . import _lib

__all__ = [
    "spgemv_forward", "spgemv_backward", "spdmm_forward", "spdmm_backward",
    "spgemm_forward", "spgemm_backward", "sptrsv_forward", "sptrsv_backward",
    "csr_transpose_forward", "csr_transpose_backward", "splincomb_forward", "splincomb_backward",
    "csr_to_dense_forward", "csr_to_dense_backward", "csr_row_sum_forward", "csr_row_sum_backward",
    "csr_extract_diagonal_forward", "csr_extract_diagonal_backward",
    "clear_plan_cache", "plan_cache_size", "sptrsv_schedule", "sptrsv_chain_levels", "sptrsv_shared_launches",
]


def _dt(t):
    if t.dtype == torch.float32:
        return _lib.NM_F32
    if t.dtype == torch.float64:
        return _lib.NM_F64
    # the reference dispatches with AT_DISPATCH_FLOATING_TYPES (cpp/sparse_csr_cpu.cpp:22)
    raise RuntimeError(f"numml_amd: values must be float32 or float64, got {t.dtype}")


def _need_device(*tensors):
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError(
            "numml_amd: this backend runs on HIP devices only; got a tensor on "
            f"'{dev}' (no CPU implementation is provided)")
    for t in tensors[1:]:
        if t.device != dev:
            devs = ", ".join(str(x.device) for x in tensors)
            raise RuntimeError(f"expected all tensors to be on the same device, but got {devs}")
    return dev


def _idx(t, name):
    if t.dtype != torch.int64:
        # the reference reads structure through accessor<int64_t, 1> (cpp/sparse_csr_cpu.cpp:24-25)
        raise RuntimeError(f"expected scalar type Long for {name} but found {t.dtype}")
    return t.contiguous()


def _same_dtype(a, b, what):
    if a.dtype != b.dtype:
        raise RuntimeError(f"expected {what} of type {a.dtype} but found {b.dtype}")


def _wanted(a, b):
    """Which of its two gradients a backward pass computes: both when neither operand requires a
    gradient (a direct call outside autograd; what the reference's CPU path gives), otherwise
    those that are required -- the reference's GPU path computes a gradient only for an operand
    that requires one (cpp/sparse_csr_cuda.cu:662, :682).  A gradient left out is returned as None."""
    ra, rb = bool(a.requires_grad), bool(getattr(b, "requires_grad", False))
    return (True, True) if not (ra or rb) else (ra, rb)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(dev):
    return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def _rowmajor(M):
    """2-D tensor with unit column stride (copied only when it is not already)."""
    if M.dim() != 2:
        raise RuntimeError(f"expected a 2-D tensor, got {M.dim()}-D")
    if M.shape[1] > 1 and M.stride(1) != 1:
        M = M.contiguous()
    if M.shape[0] > 1 and M.stride(0) < max(M.shape[1], 1):
        M = M.contiguous()
    ld = M.stride(0) if M.shape[0] > 1 else max(M.shape[1], 1)
    return M, ld


# Host-side checks of everything a kernel would index with; they look at tensor metadata
# only and run before anything is launched (a wrong length would otherwise become an
# out-of-bounds access on the device).

def _check_csr(who, rows, cols, data, indices, indptr):
    if rows < 0 or cols < 0:
        raise RuntimeError(f"{who}: negative shape {rows} x {cols}")
    if indptr.dim() != 1 or indptr.shape[0] != rows + 1:
        raise RuntimeError(f"{who}: expected {rows + 1} row pointers for {rows} rows, got a tensor of shape "
                           f"{list(indptr.shape)}")
    if data.dim() != 1 or indices.dim() != 1 or data.shape[0] != indices.shape[0]:
        raise RuntimeError(f"{who}: values and column indices must be 1-D and of equal length, got "
                           f"{list(data.shape)} and {list(indices.shape)}")


def _check_vector(who, name, t, n):
    if t.dim() != 1 or t.shape[0] != n:
        raise RuntimeError(f"{who}: expected {name} with {n} entries, got shape {list(t.shape)}")


def _check_matrix(who, name, t, rows, cols=None):
    if t.dim() != 2 or t.shape[0] != rows or (cols is not None and t.shape[1] != cols):
        raise RuntimeError(f"{who}: expected {name} of shape {rows} x {'n' if cols is None else cols}, got "
                           f"{list(t.shape)}")


def _square(who, rows, cols):
    if rows != cols:
        raise RuntimeError(f"{who}: expected a square matrix, got {rows} x {cols}")


# ------------------------------------------------------------ structure plans
#
# This module is the thin way to the C ABI (tests call the library through it); the plan
# POLICY of the package -- content keys, building a plan at the second sighting of a pattern,
# the byte-bounded cache -- lives in one place only, the compiled binding
# (csrc/torch_binding.cpp).  Here a plan is built the first time a pair of structure tensors is
# seen and kept under their identity (storage address and version counter; the plan keeps the
# tensors alive so that the address cannot be reused), at most _PLAN_CACHE_SIZE of them.

_PLAN_CACHE_SIZE = 16
_plans = collections.OrderedDict()
_plans_lock = threading.Lock()

# "planned" / "eager": backward passes walk A by column on a transposed-structure plan
#            (deterministic, no atomics);  "atomic": stateless scatter with atomics.
BACKWARD_MODE = os.environ.get("NUMML_AMD_BACKWARD", "planned")


def clear_plan_cache():
    with _plans_lock:
        _plans.clear()


# plans hold device tensors and events: given back while torch is still whole
atexit.register(clear_plan_cache)


def _cached(kind, indices, indptr, extra, make):
    key = (kind, indices.device.index, indices.data_ptr(), indptr.data_ptr(), indices._version,
           indptr._version, indices.shape[0], indptr.shape[0]) + tuple(extra)
    with _plans_lock:
        plan = _plans.get(key)
        if plan is not None:
            _plans.move_to_end(key)
            return plan
    plan = make()
    with _plans_lock:
        _plans[key] = plan
        while len(_plans) > _PLAN_CACHE_SIZE:
            _plans.popitem(last=False)
    return plan


class _TransposePlan:
    """Device arrays of the transposed structure (see nm_csr_transpose_plan_build)."""

    def __init__(self, indices, indptr, rows, cols, dev):
        L = _lib.lib()
        nnz = indices.shape[0]
        pbytes, wbytes = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _lib.check(L.nm_csr_transpose_plan_bytes(rows, cols, nnz, ctypes.byref(pbytes),
                                                 ctypes.byref(wbytes)), "nm_csr_transpose_plan_bytes")
        self.mem = torch.empty(max(pbytes.value, 8), dtype=torch.uint8, device=dev)
        work = torch.empty(max(wbytes.value, 8), dtype=torch.uint8, device=dev)
        self.indices, self.indptr = indices, indptr
        _lib.check(L.nm_csr_transpose_plan_build(
            rows, cols, nnz, _ptr(indices), _ptr(indptr), _ptr(self.mem), pbytes.value, _ptr(work),
            wbytes.value, _stream(dev)), "nm_csr_transpose_plan_build")
        self.ready = torch.cuda.Event()
        self.ready.record(torch.cuda.current_stream(dev))
        # `work` returns to torch's caching allocator, which hands it out again only to
        # work enqueued later on this same stream
        self._shape, self._info = (rows, cols, nnz), None

    def info(self, dev):
        """The plan's figures (nm_csr_transpose_plan_info), fetched once: the call waits for the
        stream."""
        if self._info is None:
            buf = (ctypes.c_int32 * 16)()
            rows, cols, nnz = self._shape
            _lib.check(_lib.lib().nm_csr_transpose_plan_info(rows, cols, nnz, _ptr(self.mem), buf, _stream(dev)),
                       "nm_csr_transpose_plan_info")
            self._info = list(buf)
        return self._info


def _fits_a_plan(rows, cols, nnz):
    """A transposed-structure plan keeps rows, columns and positions in 32 bits; larger matrices
    run the stateless kernels, which take 64-bit offsets throughout."""
    lim = 0x7ffffffe
    return rows < lim and cols < lim and nnz < lim


def _transpose_plan(indices, indptr, rows, cols, dev):
    plan = _cached("T", indices, indptr, (rows, cols),
                   lambda: _TransposePlan(indices, indptr, rows, cols, dev))
    # a plan built on another stream must have finished before this stream reads it
    torch.cuda.current_stream(dev).wait_event(plan.ready)
    return plan


# --------------------------------------------------------------------- SpMV

def spgemv_forward(A_rows, A_cols, A_data, A_col_ind, A_rowptr, x):
    """y = A x  (cpp/sparse_csr.hpp:32-36)."""
    _check_csr("spgemv_forward", A_rows, A_cols, A_data, A_col_ind, A_rowptr)
    _check_vector("spgemv_forward", "x", x, A_cols)
    dev = _need_device(A_data, A_col_ind, A_rowptr, x)
    _same_dtype(A_data, x, "x")
    A_data, x = A_data.contiguous(), x.contiguous()
    A_col_ind, A_rowptr = _idx(A_col_ind, "A_col_ind"), _idx(A_rowptr, "A_rowptr")
    if x.dim() != 1:
        raise RuntimeError(f"expected 1-D x, got {x.dim()}-D")
    with torch.cuda.device(dev):
        y = torch.empty(A_rows, dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_spgemv_forward(
            _dt(A_data), A_rows, x.shape[0], A_data.shape[0], _ptr(A_data), _ptr(A_col_ind),
            _ptr(A_rowptr), _ptr(x), _ptr(y), _stream(dev)), "nm_spgemv_forward")
    return y


def spgemv_backward(grad_z, A_rows, A_cols, A_data, A_col_ind, A_rowptr, x):
    """[grad_A, grad_x]  (cpp/sparse_csr.hpp:38-42)."""
    _check_csr("spgemv_backward", A_rows, A_cols, A_data, A_col_ind, A_rowptr)
    _check_vector("spgemv_backward", "x", x, A_cols)
    _check_vector("spgemv_backward", "grad_z", grad_z, A_rows)
    dev = _need_device(grad_z, A_data, A_col_ind, A_rowptr, x)
    _same_dtype(A_data, x, "x")
    _same_dtype(A_data, grad_z, "grad_z")
    want_A, want_x = _wanted(A_data, x)
    A_data, x, grad_z = A_data.contiguous(), x.contiguous(), grad_z.contiguous()
    A_col_ind, A_rowptr = _idx(A_col_ind, "A_col_ind"), _idx(A_rowptr, "A_rowptr")
    with torch.cuda.device(dev):
        grad_A = torch.empty_like(A_data) if want_A else None
        grad_x = torch.empty_like(x) if want_x else None
        if BACKWARD_MODE != "atomic" and _fits_a_plan(A_rows, x.shape[0], A_data.shape[0]):
            plan = _transpose_plan(A_col_ind, A_rowptr, A_rows, x.shape[0], dev)
            # most blocks of 256 columns have a staging list: the build that stages g and x in LDS
            lists = 2 * plan.info(dev)[5] >= (x.shape[0] + 255) // 256
            entry = _lib.lib().nm_spgemv_backward_planned_lists if lists else _lib.lib().nm_spgemv_backward_planned
            _lib.check(entry(
                _dt(A_data), A_rows, x.shape[0], A_data.shape[0], _ptr(A_data), _ptr(plan.mem), _ptr(x),
                _ptr(grad_z), _ptr(grad_A), _ptr(grad_x), _stream(dev)), "nm_spgemv_backward_planned")
            return [grad_A, grad_x]
        _lib.check(_lib.lib().nm_spgemv_backward(
            _dt(A_data), A_rows, x.shape[0], A_data.shape[0], _ptr(A_data), _ptr(A_col_ind),
            _ptr(A_rowptr), _ptr(x), _ptr(grad_z), _ptr(grad_A), _ptr(grad_x), _stream(dev)),
            "nm_spgemv_backward")
    return [grad_A, grad_x]


# --------------------------------------------------------------------- SpMM

def csr_transpose_forward(A_rows, A_columns, A_data, A_indices, A_indptr):
    """[At_data, At_indices, At_indptr, At_to_A_idx]  (cpp/sparse_csr.hpp:57-61)."""
    _check_csr("csr_transpose_forward", A_rows, A_columns, A_data, A_indices, A_indptr)
    dev = _need_device(A_data, A_indices, A_indptr)
    A_data = A_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    nnz = A_data.shape[0]
    with torch.cuda.device(dev):
        plan = _transpose_plan(A_indices, A_indptr, A_rows, A_columns, dev)
        At_data = torch.empty_like(A_data)
        At_indices = torch.empty(nnz, dtype=torch.int64, device=dev)
        At_indptr = torch.empty(A_columns + 1, dtype=torch.int64, device=dev)
        At_to_A = torch.empty(nnz, dtype=torch.int64, device=dev)
        _lib.check(_lib.lib().nm_csr_transpose_forward(
            _dt(A_data), A_rows, A_columns, nnz, _ptr(A_data), _ptr(plan.mem), _ptr(At_data),
            _ptr(At_indices), _ptr(At_indptr), _ptr(At_to_A), _stream(dev)), "nm_csr_transpose_forward")
    return [At_data, At_indices, At_indptr, At_to_A]


def csr_transpose_backward(grad_At, At_to_A_idx):
    """grad_A with grad_A[At_to_A_idx[p]] = grad_At[p]  (cpp/sparse_csr.hpp:63-65)."""
    _check_vector("csr_transpose_backward", "At_to_A_idx", At_to_A_idx, grad_At.numel())
    if grad_At.dim() != 1:
        raise RuntimeError(f"csr_transpose_backward: expected 1-D grad_At, got shape {list(grad_At.shape)}")
    dev = _need_device(grad_At, At_to_A_idx)
    _dt(grad_At)
    grad_At = grad_At.contiguous()
    At_to_A_idx = _idx(At_to_A_idx, "At_to_A_idx")
    with torch.cuda.device(dev):
        grad_A = torch.empty_like(grad_At)
        _lib.check(_lib.lib().nm_csr_transpose_backward(
            _dt(grad_At), grad_At.shape[0], _ptr(grad_At), _ptr(At_to_A_idx), _ptr(grad_A), _stream(dev)),
            "nm_csr_transpose_backward")
    return grad_A


def _scalar(v):
    return float(v.item()) if isinstance(v, torch.Tensor) else float(v)


def splincomb_forward(rows, cols, alpha, A_data, A_indices, A_indptr, beta, B_data, B_indices, B_indptr):
    """[C_data, C_indices, C_indptr] of alpha A + beta B  (cpp/sparse_csr.hpp:67-72)."""
    _check_csr("splincomb_forward", rows, cols, A_data, A_indices, A_indptr)
    _check_csr("splincomb_forward", rows, cols, B_data, B_indices, B_indptr)
    dev = _need_device(A_data, A_indices, A_indptr, B_data, B_indices, B_indptr)
    _same_dtype(A_data, B_data, "B_data")
    A_data, B_data = A_data.contiguous(), B_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    B_indices, B_indptr = _idx(B_indices, "B_indices"), _idx(B_indptr, "B_indptr")
    a, b = _scalar(alpha), _scalar(beta)
    L = _lib.lib()
    with torch.cuda.device(dev):
        nbytes = ctypes.c_size_t(0)
        _lib.check(L.nm_splincomb_workspace_bytes(rows, ctypes.byref(nbytes)), "nm_splincomb_workspace_bytes")
        work = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
        C_indptr = torch.empty(rows + 1, dtype=torch.int64, device=dev)
        _lib.check(L.nm_splincomb_symbolic(rows, _ptr(A_indices), _ptr(A_indptr), _ptr(B_indices), _ptr(B_indptr),
                                           _ptr(C_indptr), _ptr(work), nbytes.value, _stream(dev)),
                   "nm_splincomb_symbolic")
        nnz_c = int(C_indptr[rows].item())
        C_indices = torch.empty(nnz_c, dtype=torch.int64, device=dev)
        C_data = torch.empty(nnz_c, dtype=A_data.dtype, device=dev)
        _lib.check(L.nm_splincomb_numeric(_dt(A_data), rows, a, _ptr(A_data), _ptr(A_indices), _ptr(A_indptr), b,
                                          _ptr(B_data), _ptr(B_indices), _ptr(B_indptr), _ptr(C_indptr),
                                          _ptr(C_indices), _ptr(C_data), _stream(dev)), "nm_splincomb_numeric")
    return [C_data, C_indices, C_indptr]


def splincomb_backward(rows, cols, alpha, A_data, A_indices, A_indptr, beta, B_data, B_indices, B_indptr,
                       grad_C_data, C_indices, C_indptr):
    """[grad_A, grad_B]  (cpp/sparse_csr.hpp:74-79)."""
    _check_csr("splincomb_backward", rows, cols, A_data, A_indices, A_indptr)
    _check_csr("splincomb_backward", rows, cols, B_data, B_indices, B_indptr)
    _check_csr("splincomb_backward", rows, cols, grad_C_data, C_indices, C_indptr)
    dev = _need_device(A_data, A_indices, A_indptr, B_data, B_indices, B_indptr, grad_C_data, C_indices, C_indptr)
    _same_dtype(A_data, B_data, "B_data")
    _same_dtype(A_data, grad_C_data, "grad_C_data")
    grad_C_data = grad_C_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    B_indices, B_indptr = _idx(B_indices, "B_indices"), _idx(B_indptr, "B_indptr")
    C_indices, C_indptr = _idx(C_indices, "C_indices"), _idx(C_indptr, "C_indptr")
    a, b = _scalar(alpha), _scalar(beta)
    want_A, want_B = _wanted(A_data, B_data)
    with torch.cuda.device(dev):
        grad_A = torch.empty(A_data.shape[0], dtype=A_data.dtype, device=dev) if want_A else None
        grad_B = torch.empty(B_data.shape[0], dtype=B_data.dtype, device=dev) if want_B else None
        _lib.check(_lib.lib().nm_splincomb_backward(
            _dt(A_data), rows, a, _ptr(A_indices), _ptr(A_indptr), b, _ptr(B_indices), _ptr(B_indptr),
            _ptr(grad_C_data), _ptr(C_indices), _ptr(C_indptr), _ptr(grad_A), _ptr(grad_B), _stream(dev)),
            "nm_splincomb_backward")
    return [grad_A, grad_B]


def csr_to_dense_forward(A_rows, A_cols, A_data, A_indices, A_indptr):
    """Dense A_rows x A_cols copy  (cpp/sparse_csr.hpp:122-126)."""
    _check_csr("csr_to_dense_forward", A_rows, A_cols, A_data, A_indices, A_indptr)
    dev = _need_device(A_data, A_indices, A_indptr)
    A_data = A_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        A_d = torch.empty((A_rows, A_cols), dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_csr_to_dense_forward(
            _dt(A_data), A_rows, A_cols, A_data.shape[0], _ptr(A_data), _ptr(A_indices), _ptr(A_indptr), _ptr(A_d),
            A_cols, _stream(dev)), "nm_csr_to_dense_forward")
    return A_d


def csr_to_dense_backward(grad_Ad, A_rows, A_cols, A_data, A_indices, A_indptr):
    """grad_A[k] = grad_Ad[row(k), col(k)]  (cpp/sparse_csr.hpp:128-133)."""
    _check_csr("csr_to_dense_backward", A_rows, A_cols, A_data, A_indices, A_indptr)
    dev = _need_device(grad_Ad, A_data, A_indices, A_indptr)
    _same_dtype(A_data, grad_Ad, "grad_Ad")
    if grad_Ad.ndim != 2 or tuple(grad_Ad.shape) != (A_rows, A_cols):
        raise RuntimeError(f"expected a {A_rows} x {A_cols} gradient, got {tuple(grad_Ad.shape)}")
    grad_Ad, ld = _rowmajor(grad_Ad)
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        grad_A = torch.empty(A_data.shape[0], dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_csr_to_dense_backward(
            _dt(A_data), A_rows, A_cols, A_data.shape[0], _ptr(grad_Ad), max(ld, A_cols), _ptr(A_indices),
            _ptr(A_indptr), _ptr(grad_A), _stream(dev)), "nm_csr_to_dense_backward")
    return grad_A


def csr_row_sum_forward(A_rows, A_cols, A_data, A_indices, A_indptr):
    """x[i] = sum of row i  (cpp/sparse_csr.hpp:136-140)."""
    _check_csr("csr_row_sum_forward", A_rows, A_cols, A_data, A_indices, A_indptr)
    dev = _need_device(A_data, A_indices, A_indptr)
    A_data, A_indptr = A_data.contiguous(), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        x = torch.empty(A_rows, dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_csr_row_sum_forward(_dt(A_data), A_rows, A_data.shape[0], _ptr(A_data),
                                                     _ptr(A_indptr), _ptr(x), _stream(dev)),
                   "nm_csr_row_sum_forward")
    return x


def csr_row_sum_backward(grad_x, A_rows, A_cols, A_data, A_indices, A_indptr):
    """grad_A[k] = grad_x[row(k)]  (cpp/sparse_csr.hpp:142-147)."""
    _check_csr("csr_row_sum_backward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_vector("csr_row_sum_backward", "grad_x", grad_x, A_rows)
    dev = _need_device(grad_x, A_data, A_indices, A_indptr)
    _same_dtype(A_data, grad_x, "grad_x")
    grad_x, A_indptr = grad_x.contiguous(), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        grad_A = torch.empty(A_data.shape[0], dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_csr_row_sum_backward(_dt(A_data), A_rows, A_data.shape[0], _ptr(A_indptr),
                                                      _ptr(grad_x), _ptr(grad_A), _stream(dev)),
                   "nm_csr_row_sum_backward")
    return grad_A


def csr_extract_diagonal_forward(A_rows, A_cols, A_data, A_indices, A_indptr):
    """x[i] = stored entry (i, i) or 0  (cpp/sparse_csr.hpp:150-154)."""
    _check_csr("csr_extract_diagonal_forward", A_rows, A_cols, A_data, A_indices, A_indptr)
    dev = _need_device(A_data, A_indices, A_indptr)
    A_data = A_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        x = torch.empty(A_rows, dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_csr_extract_diagonal_forward(
            _dt(A_data), A_rows, A_data.shape[0], _ptr(A_data), _ptr(A_indices), _ptr(A_indptr), _ptr(x),
            _stream(dev)), "nm_csr_extract_diagonal_forward")
    return x


def csr_extract_diagonal_backward(grad_x, A_rows, A_cols, A_data, A_indices, A_indptr):
    """grad_A = 0 except grad_x[i] on the diagonal entries  (cpp/sparse_csr.hpp:156-161)."""
    _check_csr("csr_extract_diagonal_backward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_vector("csr_extract_diagonal_backward", "grad_x", grad_x, A_rows)
    dev = _need_device(grad_x, A_data, A_indices, A_indptr)
    _same_dtype(A_data, grad_x, "grad_x")
    grad_x = grad_x.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        grad_A = torch.empty(A_data.shape[0], dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_csr_extract_diagonal_backward(
            _dt(A_data), A_rows, A_data.shape[0], _ptr(A_indices), _ptr(A_indptr), _ptr(grad_x), _ptr(grad_A),
            _stream(dev)), "nm_csr_extract_diagonal_backward")
    return grad_A


def spdmm_forward(A_rows, A_cols, A_data, A_indices, A_indptr, B):
    """C = A B, B dense 2-D  (cpp/sparse_csr.hpp:81-85)."""
    _check_csr("spdmm_forward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_matrix("spdmm_forward", "B", B, A_cols)
    dev = _need_device(A_data, A_indices, A_indptr, B)
    _same_dtype(A_data, B, "B")
    A_data = A_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    B, ldb = _rowmajor(B)
    n = B.shape[1]
    with torch.cuda.device(dev):
        C = torch.empty((A_rows, n), dtype=A_data.dtype, device=dev)
        _lib.check(_lib.lib().nm_spdmm_forward(
            _dt(A_data), A_rows, B.shape[0], A_data.shape[0], _ptr(A_data), _ptr(A_indices),
            _ptr(A_indptr), _ptr(B), ldb, n, _ptr(C), max(n, 1), _stream(dev)), "nm_spdmm_forward")
    return C


def spdmm_backward(A_rows, A_cols, A_data, A_indices, A_indptr, B, grad_C):
    """[grad_A, grad_B]  (cpp/sparse_csr.hpp:87-91)."""
    _check_csr("spdmm_backward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_matrix("spdmm_backward", "B", B, A_cols)
    _check_matrix("spdmm_backward", "grad_C", grad_C, A_rows, B.shape[1])
    dev = _need_device(A_data, A_indices, A_indptr, B, grad_C)
    _same_dtype(A_data, B, "B")
    _same_dtype(A_data, grad_C, "grad_C")
    want_A, want_B = _wanted(A_data, B)
    A_data = A_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    B, ldb = _rowmajor(B)
    grad_C, ldg = _rowmajor(grad_C)
    n = B.shape[1]
    with torch.cuda.device(dev):
        grad_A = torch.empty_like(A_data) if want_A else None
        grad_B = torch.empty((B.shape[0], n), dtype=B.dtype, device=dev) if want_B else None
        if want_B and BACKWARD_MODE != "atomic" and _fits_a_plan(A_rows, B.shape[0], A_data.shape[0]):
            plan = _transpose_plan(A_indices, A_indptr, A_rows, B.shape[0], dev)
            _lib.check(_lib.lib().nm_spdmm_backward_planned(
                _dt(A_data), A_rows, B.shape[0], A_data.shape[0], _ptr(A_data), _ptr(A_indices),
                _ptr(A_indptr), _ptr(plan.mem), _ptr(B), ldb, _ptr(grad_C), ldg, n, _ptr(grad_A),
                _ptr(grad_B), max(n, 1), _stream(dev)), "nm_spdmm_backward_planned")
            return [grad_A, grad_B]
        _lib.check(_lib.lib().nm_spdmm_backward(
            _dt(A_data), A_rows, B.shape[0], A_data.shape[0], _ptr(A_data), _ptr(A_indices),
            _ptr(A_indptr), _ptr(B), ldb, _ptr(grad_C), ldg, n, _ptr(grad_A), _ptr(grad_B),
            max(n, 1), _stream(dev)), "nm_spdmm_backward")
    return [grad_A, grad_B]


# ------------------------------------------------------------------- SpGEMM

_landing = threading.local()


def _host_landing():
    """32 bytes of pinned host memory per host thread: where nm_spgemm_symbolic_result has the
    device drop nnz(C) (torch's pinned-memory allocator owns it)."""
    t = getattr(_landing, "t", None)
    if t is None:
        t = _landing.t = torch.zeros(4, dtype=torch.int64).pin_memory()
    return t


def spgemm_forward(A_rows, A_cols, A_data, A_indices, A_indptr,
                   B_rows, B_cols, B_data, B_indices, B_indptr):
    """[C_data, C_indices, C_indptr]  (cpp/sparse_csr.hpp:45-48).

    One device->host read of nnz(C) sits between the two phases; it is inherent
    to the interface, which returns exactly-sized tensors.
    """
    _check_csr("spgemm_forward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_csr("spgemm_forward", B_rows, B_cols, B_data, B_indices, B_indptr)
    if A_cols != B_rows:
        raise RuntimeError(f"spgemm_forward: A has {A_cols} columns but B has {B_rows} rows")
    dev = _need_device(A_data, A_indices, A_indptr, B_data, B_indices, B_indptr)
    _same_dtype(A_data, B_data, "B_data")
    A_data, B_data = A_data.contiguous(), B_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    B_indices, B_indptr = _idx(B_indices, "B_indices"), _idx(B_indptr, "B_indptr")
    L = _lib.lib()
    with torch.cuda.device(dev):
        nbytes = ctypes.c_size_t(0)
        _lib.check(L.nm_spgemm_workspace_bytes(A_rows, B_cols, ctypes.byref(nbytes)),
                   "nm_spgemm_workspace_bytes")
        work = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
        C_indptr = torch.empty(A_rows + 1, dtype=torch.int64, device=dev)
        st = _stream(dev)
        _lib.check(L.nm_spgemm_symbolic(
            A_rows, A_cols, B_cols, _ptr(A_indices), _ptr(A_indptr), _ptr(B_indices), _ptr(B_indptr),
            _ptr(C_indptr), _ptr(work), nbytes.value, _ptr(_host_landing()), st), "nm_spgemm_symbolic")
        nnz_c, hash_rows = ctypes.c_int64(0), ctypes.c_int64(0)
        _lib.check(L.nm_spgemm_symbolic_result(A_rows, B_cols, _ptr(work), nbytes.value, ctypes.byref(nnz_c),
                                               ctypes.byref(hash_rows), _ptr(_host_landing()), st),
                   "nm_spgemm_symbolic_result")
        C_indices = torch.empty(nnz_c.value, dtype=torch.int64, device=dev)
        C_data = torch.empty(nnz_c.value, dtype=A_data.dtype, device=dev)
        _lib.check(L.nm_spgemm_numeric(
            _dt(A_data), A_rows, A_cols, B_cols, _ptr(A_data), _ptr(A_indices), _ptr(A_indptr),
            _ptr(B_data), _ptr(B_indices), _ptr(B_indptr), _ptr(C_indptr), _ptr(C_indices),
            _ptr(C_data), _ptr(work), nbytes.value, hash_rows.value, st), "nm_spgemm_numeric")
    return [C_data, C_indices, C_indptr]


def spgemm_backward(grad_C, C_indices, C_indptr,
                    A_rows, A_cols, A_data, A_indices, A_indptr,
                    B_rows, B_cols, B_data, B_indices, B_indptr):
    """[grad_A, grad_B]  (cpp/sparse_csr.hpp:50-54)."""
    _check_csr("spgemm_backward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_csr("spgemm_backward", B_rows, B_cols, B_data, B_indices, B_indptr)
    _check_csr("spgemm_backward", A_rows, B_cols, grad_C, C_indices, C_indptr)
    if A_cols != B_rows:
        raise RuntimeError(f"spgemm_backward: A has {A_cols} columns but B has {B_rows} rows")
    dev = _need_device(grad_C, C_indices, C_indptr, A_data, A_indices, A_indptr,
                       B_data, B_indices, B_indptr)
    _same_dtype(A_data, B_data, "B_data")
    _same_dtype(A_data, grad_C, "grad_C")
    want_A, want_B = _wanted(A_data, B_data)
    A_data, B_data, grad_C = A_data.contiguous(), B_data.contiguous(), grad_C.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    B_indices, B_indptr = _idx(B_indices, "B_indices"), _idx(B_indptr, "B_indptr")
    C_indices, C_indptr = _idx(C_indices, "C_indices"), _idx(C_indptr, "C_indptr")
    with torch.cuda.device(dev):
        grad_A = torch.empty_like(A_data) if want_A else None
        grad_B = torch.empty_like(B_data) if want_B else None
        if BACKWARD_MODE != "atomic" and _fits_a_plan(A_rows, A_cols, A_data.shape[0]):
            plan = _transpose_plan(A_indices, A_indptr, A_rows, A_cols, dev)
            _lib.check(_lib.lib().nm_spgemm_backward_planned(
                _dt(A_data), A_rows, A_cols, A_data.shape[0], B_data.shape[0], grad_C.shape[0], _ptr(grad_C),
                _ptr(C_indices), _ptr(C_indptr), _ptr(A_data), _ptr(plan.mem), _ptr(B_data), _ptr(B_indices),
                _ptr(B_indptr), _ptr(grad_A), _ptr(grad_B), _stream(dev)), "nm_spgemm_backward_planned")
            return [grad_A, grad_B]
        _lib.check(_lib.lib().nm_spgemm_backward(
            _dt(A_data), A_rows, A_data.shape[0], B_data.shape[0], _ptr(grad_C), _ptr(C_indices),
            _ptr(C_indptr), _ptr(A_data), _ptr(A_indices), _ptr(A_indptr), _ptr(B_data),
            _ptr(B_indices), _ptr(B_indptr), _ptr(grad_A), _ptr(grad_B), _stream(dev)),
            "nm_spgemm_backward")
    return [grad_A, grad_B]


def spgemm_forward_mapped(A_rows, A_cols, A_data, A_indices, A_indptr,
                          B_rows, B_cols, B_data, B_indices, B_indptr):
    """[C_data, C_indices, C_indptr, plan]: spgemm_forward through nm_spgemm_symbolic_mapped /
    nm_spgemm_numeric_mapped, which compute the product on the destination records that the
    symbolic merge leaves behind, and the ProductPlan those records make (its ``usable`` is False
    when the product has rows on the hash path or the plan's limits do not hold)."""
    _check_csr("spgemm_forward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_csr("spgemm_forward", B_rows, B_cols, B_data, B_indices, B_indptr)
    if A_cols != B_rows:
        raise RuntimeError(f"spgemm_forward: A has {A_cols} columns but B has {B_rows} rows")
    dev = _need_device(A_data, A_indices, A_indptr, B_data, B_indices, B_indptr)
    _same_dtype(A_data, B_data, "B_data")
    A_data, B_data = A_data.contiguous(), B_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    B_indices, B_indptr = _idx(B_indices, "B_indices"), _idx(B_indptr, "B_indptr")
    L = _lib.lib()
    A_nnz, B_nnz = A_indices.shape[0], B_indices.shape[0]
    with torch.cuda.device(dev):
        nbytes, pbytes = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _lib.check(L.nm_spgemm_workspace_bytes(A_rows, B_cols, ctypes.byref(nbytes)),
                   "nm_spgemm_workspace_bytes")
        _lib.check(L.nm_spgemm_plan_bytes(A_nnz, ctypes.byref(pbytes)), "nm_spgemm_plan_bytes")
        work = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
        mem = torch.empty(max(pbytes.value, 8), dtype=torch.uint8, device=dev)
        C_indptr = torch.empty(A_rows + 1, dtype=torch.int64, device=dev)
        st = _stream(dev)
        _lib.check(L.nm_spgemm_symbolic_mapped(
            A_rows, A_cols, B_cols, A_nnz, B_nnz, _ptr(A_indices), _ptr(A_indptr), _ptr(B_indices),
            _ptr(B_indptr), _ptr(C_indptr), _ptr(work), nbytes.value, _ptr(mem), pbytes.value,
            _ptr(_host_landing()), st), "nm_spgemm_symbolic_mapped")
        nnz_c, hash_rows = ctypes.c_int64(0), ctypes.c_int64(0)
        _lib.check(L.nm_spgemm_symbolic_result(A_rows, B_cols, _ptr(work), nbytes.value, ctypes.byref(nnz_c),
                                               ctypes.byref(hash_rows), _ptr(_host_landing()), st),
                   "nm_spgemm_symbolic_result")
        C_indices = torch.empty(nnz_c.value, dtype=torch.int64, device=dev)
        C_data = torch.empty(nnz_c.value, dtype=A_data.dtype, device=dev)
        _lib.check(L.nm_spgemm_numeric_mapped(
            _dt(A_data), A_rows, A_cols, B_cols, A_nnz, nnz_c.value, _ptr(A_data), _ptr(A_indices),
            _ptr(A_indptr), _ptr(B_data), _ptr(B_indices), _ptr(B_indptr), _ptr(C_indptr), _ptr(C_indices),
            _ptr(C_data), _ptr(work), nbytes.value, hash_rows.value, _ptr(mem), pbytes.value, 1, st),
            "nm_spgemm_numeric_mapped")
        plan = ProductPlan(A_rows, A_cols, A_indices, A_indptr, B_indices, B_indptr, C_indices, C_indptr,
                           adopt=(mem, hash_rows.value))
    return [C_data, C_indices, C_indptr, plan]


class ProductPlan:
    """Product plan of C = A B (nm_spgemm_plan_build): numeric product and gradients of a product
    whose three patterns are known, without the symbolic phase and without searches.

    ``usable`` is False when a row is longer than the plan's limits; then neither method may be
    called.  The plan keeps the structure tensors it was built from alive.  With ``adopt`` =
    (plan memory filled by a mapped forward pass, its hash_rows) nothing is built: the memory is
    checked (nm_spgemm_plan_adopt) and taken over.
    """

    def __init__(self, A_rows, A_cols, A_indices, A_indptr, B_indices, B_indptr, C_indices, C_indptr, adopt=None):
        dev = _need_device(A_indices, A_indptr, B_indices, B_indptr, C_indices, C_indptr)
        L = _lib.lib()
        self.dev, self.A_rows, self.A_cols = dev, A_rows, A_cols
        self.A_nnz, self.B_nnz, self.C_nnz = A_indices.shape[0], B_indices.shape[0], C_indices.shape[0]
        self.A_indptr, self.B_indptr, self.C_indptr, self.C_indices = A_indptr, B_indptr, C_indptr, C_indices
        with torch.cuda.device(dev):
            self.transposed = _transpose_plan(A_indices, A_indptr, A_rows, A_cols, dev)
            nbytes = ctypes.c_size_t(0)
            _lib.check(L.nm_spgemm_plan_bytes(self.A_nnz, ctypes.byref(nbytes)), "nm_spgemm_plan_bytes")
            usable = ctypes.c_int(0)
            if adopt is not None:
                self.mem, hash_rows = adopt
                _lib.check(L.nm_spgemm_plan_adopt(
                    A_rows, A_cols, self.A_nnz, self.B_nnz, self.C_nnz, hash_rows, _ptr(self.transposed.mem),
                    _ptr(self.mem), nbytes.value, _ptr(_host_landing()), ctypes.byref(usable), _stream(dev)),
                    "nm_spgemm_plan_adopt")
                self.usable, self.plan_class = usable.value > 0, usable.value
                return
            self.mem = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
            _lib.check(L.nm_spgemm_plan_build(
                A_rows, A_cols, self.A_nnz, self.B_nnz, self.C_nnz, _ptr(A_indices), _ptr(A_indptr),
                _ptr(B_indices), _ptr(B_indptr), _ptr(C_indices), _ptr(C_indptr), _ptr(self.transposed.mem),
                _ptr(self.mem), nbytes.value, _ptr(_host_landing()), ctypes.byref(usable), _stream(dev)),
                "nm_spgemm_plan_build")
            if usable.value < 0:
                # the only obstacle is the length of the rows of B that A names (9 to 32 entries):
                # a plan with two or four destination octets per entry of A
                octets = 2 if -usable.value <= 16 else 4
                _lib.check(L.nm_spgemm_plan_bytes_wide(self.A_nnz, octets, ctypes.byref(nbytes)),
                           "nm_spgemm_plan_bytes_wide")
                self.mem = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
                _lib.check(L.nm_spgemm_plan_build_wide(
                    A_rows, A_cols, self.A_nnz, self.B_nnz, self.C_nnz, _ptr(A_indices), _ptr(A_indptr),
                    _ptr(B_indices), _ptr(B_indptr), _ptr(C_indices), _ptr(C_indptr), _ptr(self.transposed.mem),
                    _ptr(self.mem), nbytes.value, octets, _ptr(_host_landing()), ctypes.byref(usable), _stream(dev)),
                    "nm_spgemm_plan_build_wide")
            self.usable, self.plan_class = usable.value > 0, usable.value

    def numeric(self, A_data, B_data):
        """C_data of the product (the pattern is the one the plan was built from)."""
        if not self.usable:
            raise RuntimeError("this product has rows beyond the plan's limits")
        A_data, B_data = A_data.contiguous(), B_data.contiguous()
        with torch.cuda.device(self.dev):
            C_data = torch.empty(self.C_nnz, dtype=A_data.dtype, device=self.dev)
            _lib.check(_lib.lib().nm_spgemm_numeric_planned(
                _dt(A_data), self.plan_class, self.A_rows, self.A_nnz, self.B_nnz, self.C_nnz, _ptr(A_data),
                _ptr(self.A_indptr),
                _ptr(B_data), _ptr(self.mem), _ptr(self.C_indptr), _ptr(C_data), _stream(self.dev)),
                "nm_spgemm_numeric_planned")
        return C_data

    def backward(self, grad_C, A_data, B_data):
        """[grad_A, grad_B] of grad_C laid out on the plan's pattern of C."""
        if not self.usable:
            raise RuntimeError("this product has rows beyond the plan's limits")
        A_data, B_data, grad_C = A_data.contiguous(), B_data.contiguous(), grad_C.contiguous()
        with torch.cuda.device(self.dev):
            grad_A, grad_B = torch.empty_like(A_data), torch.empty_like(B_data)
            _lib.check(_lib.lib().nm_spgemm_backward_mapped_wide(
                _dt(A_data), self.plan_class, self.A_rows, self.A_cols, self.A_nnz, self.B_nnz, self.C_nnz,
                _ptr(grad_C), _ptr(A_data), _ptr(self.transposed.mem), _ptr(B_data), _ptr(self.B_indptr),
                _ptr(self.mem), _ptr(grad_A), _ptr(grad_B), _stream(self.dev)), "nm_spgemm_backward_mapped_wide")
        return [grad_A, grad_B]


# ------------------------------------------------------------------- SpTRSV

class _Plan:
    """Level schedule + transposed structure of one triangular sparsity pattern."""

    def __init__(self, indices, indptr, rows, lower, dev):
        L = _lib.lib()
        nnz = indices.shape[0]
        pbytes, wbytes = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _lib.check(L.nm_sptrsv_plan_bytes(rows, nnz, ctypes.byref(pbytes), ctypes.byref(wbytes)),
                   "nm_sptrsv_plan_bytes")
        self.mem = torch.empty(max(pbytes.value, 8), dtype=torch.uint8, device=dev)
        work = torch.empty(max(wbytes.value, 8), dtype=torch.uint8, device=dev)
        # the tensors are kept so that their addresses cannot be reused while the plan is cached
        self.indices, self.indptr = indices, indptr
        handle = ctypes.c_void_p(0)
        _lib.check(L.nm_sptrsv_analyse(
            rows, nnz, _ptr(indices), _ptr(indptr), int(lower), _ptr(self.mem), pbytes.value,
            _ptr(work), wbytes.value, ctypes.byref(handle), _stream(dev)), "nm_sptrsv_analyse")
        self.handle = handle
        self.levels = int(L.nm_sptrsv_plan_levels(handle))
        self.launches = int(L.nm_sptrsv_plan_launches(handle))
        self.chain_levels = (int(L.nm_sptrsv_plan_chain_levels(handle, 0)),
                             int(L.nm_sptrsv_plan_chain_levels(handle, 1)))
        self.shared_launches = (int(L.nm_sptrsv_plan_shared_launches(handle, 0)),
                                int(L.nm_sptrsv_plan_shared_launches(handle, 1)))
        # nm_sptrsv_analyse synchronised its stream, so the plan is complete for every stream

    def __del__(self):
        try:
            if getattr(self, "handle", None):
                _lib.lib().nm_sptrsv_plan_destroy(self.handle)
                self.handle = None
        except Exception:
            pass


def _plan_for(indices, indptr, rows, lower, dev):
    return _cached("L", indices, indptr, (rows, bool(lower)),
                   lambda: _Plan(indices, indptr, rows, lower, dev))


class _LUPattern:
    """Filled pattern of the LU factors of one sparsity pattern, its transpose and the map
    between them.  Every splu call on that pattern hands out these same index tensors, so the
    solves that follow find their level schedules cached."""

    def __init__(self, A_indices, A_indptr, rows, dev):
        L = _lib.lib()
        stream = _stream(dev)
        self.indices, self.indptr = A_indices, A_indptr
        nbytes = ctypes.c_size_t(0)
        _lib.check(L.nm_splu_symbolic_bytes(rows, ctypes.byref(nbytes)), "nm_splu_symbolic_bytes")
        work = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
        M_indptr = torch.empty(rows + 1, dtype=torch.int64, device=dev)
        _lib.check(L.nm_splu_symbolic(rows, _ptr(A_indices), _ptr(A_indptr), _ptr(M_indptr), _ptr(work),
                                      nbytes.value, stream), "nm_splu_symbolic")
        nnz = int(M_indptr[rows].item())
        M_indices = torch.empty(nnz, dtype=torch.int64, device=dev)
        zeros = torch.zeros(max(A_indices.shape[0], 1), dtype=torch.float32, device=dev)
        As_data = torch.empty(nnz, dtype=torch.float32, device=dev)
        _lib.check(L.nm_splu_fill(_dt(zeros), rows, _ptr(zeros), _ptr(A_indices), _ptr(A_indptr),
                                  _ptr(M_indptr), _ptr(M_indices), _ptr(As_data), _ptr(work), nbytes.value,
                                  stream), "nm_splu_fill")
        _, Mt_indices, Mt_indptr, Mt_to_M = csr_transpose_forward(rows, rows, As_data, M_indices, M_indptr)
        self.derived = (M_indices, M_indptr, Mt_indices, Mt_indptr, Mt_to_M)
        self.versions = tuple(t._version for t in self.derived)
        torch.cuda.current_stream(dev).synchronize()    # complete for every stream

    def intact(self):
        return tuple(t._version for t in self.derived) == self.versions


def _lu_pattern(A_indices, A_indptr, rows, dev):
    make = lambda: _LUPattern(A_indices, A_indptr, rows, dev)
    plan = _cached("U", A_indices, A_indptr, (rows,), make)
    if not plan.intact():      # a caller edited the tensors it was handed: build them again
        with _plans_lock:
            for key in [k for k, v in _plans.items() if v is plan]:
                del _plans[key]
        plan = _cached("U", A_indices, A_indptr, (rows,), make)
    return plan


def splu(A_rows, A_cols, A_data, A_indices, A_indptr):
    """[M_data, M_indices, M_indptr, Mt_data, Mt_indices, Mt_indptr]: L + U without pivoting on the
    filled pattern, and its transpose  (cpp/sparse_csr.hpp:107-111)."""
    _check_csr("splu", A_rows, A_cols, A_data, A_indices, A_indptr)
    dev = _need_device(A_data, A_indices, A_indptr)
    if A_rows != A_cols:
        raise RuntimeError(f"Expected square matrix for LU factorization, got {A_rows} x {A_cols}.")
    A_data = A_data.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    L = _lib.lib()
    rows = A_rows
    with torch.cuda.device(dev):
        stream = _stream(dev)
        M_indices, M_indptr, Mt_indices, Mt_indptr, Mt_to_M = _lu_pattern(A_indices, A_indptr, rows, dev).derived
        nnz = M_indices.shape[0]
        # A's values on the filled pattern, moved to the transpose: the factorisation runs by column
        As_data = torch.empty(nnz, dtype=A_data.dtype, device=dev)
        _lib.check(L.nm_splu_values(_dt(A_data), rows, _ptr(A_data), _ptr(A_indices), _ptr(A_indptr),
                                    _ptr(M_indptr), _ptr(M_indices), _ptr(As_data), stream), "nm_splu_values")
        Mt_data = csr_transpose_forward(rows, rows, As_data, M_indices, M_indptr)[0]
        nbytes = ctypes.c_size_t(0)
        _lib.check(L.nm_splu_numeric_bytes(rows, ctypes.byref(nbytes)), "nm_splu_numeric_bytes")
        work = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
        _lib.check(L.nm_splu_numeric(_dt(A_data), rows, _ptr(Mt_data), _ptr(Mt_indices), _ptr(Mt_indptr),
                                     _ptr(work), nbytes.value, 0, stream), "nm_splu_numeric")
        M_data = csr_transpose_backward(Mt_data, Mt_to_M)
    return [M_data, M_indices, M_indptr, Mt_data, Mt_indices, Mt_indptr]


def spsolve_backward(grad_x, x, A_rows, A_cols, Mt_data, Mt_indices, Mt_indptr, A_data, A_indices, A_indptr):
    """[grad_A, grad_b]: grad_b = A^-T grad_x by two solves with M^T, grad_A = -(grad_b x^T) on A's
    pattern  (cpp/sparse_csr.hpp:113-118, cpp/sparse_csr_cpu.cpp:1018-1048)."""
    _check_csr("spsolve_backward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _check_csr("spsolve_backward", A_rows, A_cols, Mt_data, Mt_indices, Mt_indptr)
    _square("spsolve_backward", A_rows, A_cols)
    _check_vector("spsolve_backward", "grad_x", grad_x, A_rows)
    _check_vector("spsolve_backward", "x", x, A_rows)
    dev = _need_device(grad_x, x, Mt_data, Mt_indices, Mt_indptr, A_data, A_indices, A_indptr)
    _same_dtype(A_data, grad_x, "grad_x")
    _same_dtype(A_data, x, "x")
    _same_dtype(A_data, Mt_data, "Mt_data")
    Mt_data, A_data, grad_x, x = Mt_data.contiguous(), A_data.contiguous(), grad_x.contiguous(), x.contiguous()
    Mt_indices, Mt_indptr = _idx(Mt_indices, "Mt_indices"), _idx(Mt_indptr, "Mt_indptr")
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        lower = _plan_for(Mt_indices, Mt_indptr, A_rows, True, dev)
        y = _solve(lower, False, Mt_data, Mt_indices, Mt_indptr, False, grad_x, A_rows, dev)
        upper = _plan_for(Mt_indices, Mt_indptr, A_rows, False, dev)
        grad_b = _solve(upper, False, Mt_data, Mt_indices, Mt_indptr, True, y, A_rows, dev)
        grad_A = torch.empty_like(A_data)
        _lib.check(_lib.lib().nm_masked_outer(
            _dt(A_data), A_rows, A_data.shape[0], _ptr(A_indices), _ptr(A_indptr), -1.0,
            _ptr(grad_b), _ptr(x), _ptr(grad_A), _stream(dev)), "nm_masked_outer")
    return [grad_A, grad_b]


def sptrsv_schedule(A_rows, A_indices, A_indptr, lower):
    """(dependency levels, kernel launches per solve) of the level schedule of a
    triangular pattern, built or taken from the cache; diagnostics, no counterpart
    in the reference."""
    if A_indptr.dim() != 1 or A_indptr.shape[0] != A_rows + 1 or A_indices.dim() != 1:
        raise RuntimeError(f"sptrsv_schedule: expected {A_rows + 1} row pointers, got shape {list(A_indptr.shape)}")
    dev = _need_device(A_indices, A_indptr)
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        plan = _plan_for(A_indices, A_indptr, A_rows, lower, dev)
    return plan.levels, plan.launches


def sptrsv_chain_levels(A_rows, A_indices, A_indptr, lower):
    """Levels of the solve with A and of the solve with A^T that the single-wavefront chain
    kernels take (runs of one-row levels); diagnostics, no counterpart in the reference."""
    if A_indptr.dim() != 1 or A_indptr.shape[0] != A_rows + 1 or A_indices.dim() != 1:
        raise RuntimeError(f"sptrsv_chain_levels: expected {A_rows + 1} row pointers, got shape {list(A_indptr.shape)}")
    dev = _need_device(A_indices, A_indptr)
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        plan = _plan_for(A_indices, A_indptr, A_rows, lower, dev)
    return plan.chain_levels


def sptrsv_shared_launches(A_rows, A_indices, A_indptr, lower):
    """Launches of the solve with A and of the solve with A^T whose levels several workgroups
    share; diagnostics, no counterpart in the reference."""
    if A_indptr.dim() != 1 or A_indptr.shape[0] != A_rows + 1 or A_indices.dim() != 1:
        raise RuntimeError(f"sptrsv_shared_launches: expected {A_rows + 1} row pointers, got shape {list(A_indptr.shape)}")
    dev = _need_device(A_indices, A_indptr)
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        plan = _plan_for(A_indices, A_indptr, A_rows, lower, dev)
    return plan.shared_launches


def plan_cache_size():
    with _plans_lock:
        return len(_plans)


def _solve(plan, transposed, A_data, A_indices, A_indptr, unit, b, rows, dev):
    L = _lib.lib()
    x = torch.empty(rows, dtype=A_data.dtype, device=dev)
    nbytes = ctypes.c_size_t(0)
    _lib.check(L.nm_sptrsv_solve_bytes(rows, A_data.shape[0], ctypes.byref(nbytes)), "nm_sptrsv_solve_bytes")
    work = torch.empty(max(nbytes.value, 8), dtype=torch.uint8, device=dev)
    _lib.check(L.nm_sptrsv_solve(
        plan.handle, _dt(A_data), int(transposed), _ptr(A_data), int(unit), _ptr(b), _ptr(x), _ptr(work),
        nbytes.value, _stream(dev)), "nm_sptrsv_solve")
    return x


def sptrsv_forward(A_rows, A_cols, A_data, A_indices, A_indptr, lower, unit, b):
    """x = A^{-1} b for triangular A  (cpp/sparse_csr.hpp:94-98)."""
    _check_csr("sptrsv_forward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _square("sptrsv_forward", A_rows, A_cols)
    _check_vector("sptrsv_forward", "b", b, A_rows)
    dev = _need_device(A_data, A_indices, A_indptr, b)
    _same_dtype(A_data, b, "b")
    A_data, b = A_data.contiguous(), b.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        plan = _plan_for(A_indices, A_indptr, A_rows, lower, dev)
        return _solve(plan, False, A_data, A_indices, A_indptr, unit, b, A_rows, dev)


def sptrsv_backward(grad_x, x, A_rows, A_cols, A_data, A_indices, A_indptr, lower, unit, b):
    """[grad_A, grad_b]  (cpp/sparse_csr.hpp:100-105)."""
    _check_csr("sptrsv_backward", A_rows, A_cols, A_data, A_indices, A_indptr)
    _square("sptrsv_backward", A_rows, A_cols)
    _check_vector("sptrsv_backward", "grad_x", grad_x, A_rows)
    _check_vector("sptrsv_backward", "x", x, A_rows)
    dev = _need_device(grad_x, x, A_data, A_indices, A_indptr)
    _same_dtype(A_data, grad_x, "grad_x")
    _same_dtype(A_data, x, "x")
    want_A, want_b = _wanted(A_data, b)
    A_data, grad_x, x = A_data.contiguous(), grad_x.contiguous(), x.contiguous()
    A_indices, A_indptr = _idx(A_indices, "A_indices"), _idx(A_indptr, "A_indptr")
    with torch.cuda.device(dev):
        plan = _plan_for(A_indices, A_indptr, A_rows, lower, dev)
        # (grad_A is formed from grad_b, so the transposed solve runs whichever gradient is wanted)
        grad_b = _solve(plan, True, A_data, A_indices, A_indptr, unit, grad_x, A_rows, dev)
        if not want_A:
            return [None, grad_b]
        grad_A = torch.empty_like(A_data)
        _lib.check(_lib.lib().nm_masked_outer(
            _dt(A_data), A_rows, A_data.shape[0], _ptr(A_indices), _ptr(A_indptr), -1.0,
            _ptr(grad_b), _ptr(x), _ptr(grad_A), _stream(dev)), "nm_masked_outer")
    return [grad_A, grad_b if want_b else None]
