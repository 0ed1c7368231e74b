"""NumPy front end of liboracle.so, the serial CPU restatement of the reference.

TEST INFRASTRUCTURE ONLY.  Only tests/, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of bench.py may import this package; the product
(numml_amd/) never does.  Each function takes and returns NumPy arrays
(float32 or float64 values, int64 structure) and follows the reference CPU
function named in its docstring (paths relative to the reference tree).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    args = ["make", "-C", _HERE, "all"]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            subprocess.run(["make", "-C", _HERE, "oracle"], check=True,
                           stdout=subprocess.DEVNULL)
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.or_spgemm_symbolic.restype = ctypes.c_int64
    return _lib


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(f"oracle supports float32/float64 values, got {dtype}")


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _i64(v):
    return ctypes.c_int64(int(v))


def _vals(a, dtype=None):
    a = np.ascontiguousarray(a)
    return a if dtype is None else np.ascontiguousarray(a, dtype=dtype)


def _idx(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _fn(name, dtype):
    return getattr(lib(), f"{name}_{_sfx(dtype)}")


def spgemv_forward(rows, cols, data, indices, indptr, x):
    """spgemv_forward_cpu, cpp/sparse_csr_cpu.cpp:11-39."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    x = _vals(x, data.dtype)
    y = np.empty(rows, dtype=data.dtype)
    _fn("or_spgemv_forward", data.dtype)(_i64(rows), _p(data), _p(indices), _p(indptr), _p(x), _p(y))
    return y


def spgemv_backward(g, rows, cols, data, indices, indptr, x):
    """spgemv_backward_cpu, cpp/sparse_csr_cpu.cpp:41-77 -> (grad_A, grad_x)."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    x, g = _vals(x, data.dtype), _vals(g, data.dtype)
    grad_A = np.empty_like(data)
    grad_x = np.empty(x.shape[0], dtype=data.dtype)
    _fn("or_spgemv_backward", data.dtype)(_i64(rows), _i64(x.shape[0]), _p(data), _p(indices),
                                          _p(indptr), _p(x), _p(g), _p(grad_A), _p(grad_x))
    return grad_A, grad_x


def spdmm_forward(rows, cols, data, indices, indptr, B):
    """spdmm_forward_cpu, cpp/sparse_csr_cpu.cpp:562-602."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    B = _vals(B, data.dtype)
    n = B.shape[1]
    C = np.empty((rows, n), dtype=data.dtype)
    _fn("or_spdmm_forward", data.dtype)(_i64(rows), _p(data), _p(indices), _p(indptr), _p(B),
                                        _i64(n), _p(C))
    return C


def spdmm_backward(rows, cols, data, indices, indptr, B, gC):
    """spdmm_backward_cpu, cpp/sparse_csr_cpu.cpp:604-650 -> (grad_A, grad_B)."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    B, gC = _vals(B, data.dtype), _vals(gC, data.dtype)
    n = B.shape[1]
    grad_A = np.empty_like(data)
    grad_B = np.empty_like(B)
    _fn("or_spdmm_backward", data.dtype)(_i64(rows), _i64(B.shape[0]), _p(data), _p(indices),
                                         _p(indptr), _p(B), _p(gC), _i64(n), _p(grad_A), _p(grad_B))
    return grad_A, grad_B


def spgemm_forward(A_rows, A_cols, A_data, A_indices, A_indptr,
                   B_rows, B_cols, B_data, B_indices, B_indptr):
    """spgemm_forward_cpu, cpp/sparse_csr_cpu.cpp:117-216 -> (C_data, C_indices, C_indptr)."""
    A_data, A_indices, A_indptr = _vals(A_data), _idx(A_indices), _idx(A_indptr)
    B_data, B_indices, B_indptr = _vals(B_data, A_data.dtype), _idx(B_indices), _idx(B_indptr)
    tmp_len = max(A_rows, A_cols, B_cols, 1)
    mark = np.full(tmp_len, -1, dtype=np.int64)
    C_indptr = np.empty(A_rows + 1, dtype=np.int64)
    nnz = lib().or_spgemm_symbolic(_i64(A_rows), _p(A_indices), _p(A_indptr), _p(B_indices),
                                   _p(B_indptr), _p(C_indptr), _p(mark))
    C_indices = np.zeros(nnz, dtype=np.int64)
    C_data = np.zeros(nnz, dtype=A_data.dtype)
    mark[:] = -1
    acc = np.zeros(tmp_len, dtype=A_data.dtype)
    _fn("or_spgemm_numeric", A_data.dtype)(_i64(A_rows), _p(A_data), _p(A_indices), _p(A_indptr),
                                           _p(B_data), _p(B_indices), _p(B_indptr), _p(C_indptr),
                                           _p(C_indices), _p(C_data), _p(mark), _p(acc))
    return C_data, C_indices, C_indptr


def spgemm_backward(gC, C_indices, C_indptr,
                    A_rows, A_cols, A_data, A_indices, A_indptr,
                    B_rows, B_cols, B_data, B_indices, B_indptr):
    """spgemm_backward_cpu, cpp/sparse_csr_cpu.cpp:218-307 -> (grad_A, grad_B)."""
    A_data, A_indices, A_indptr = _vals(A_data), _idx(A_indices), _idx(A_indptr)
    B_data, B_indices, B_indptr = _vals(B_data, A_data.dtype), _idx(B_indices), _idx(B_indptr)
    gC, C_indices, C_indptr = _vals(gC, A_data.dtype), _idx(C_indices), _idx(C_indptr)
    grad_A = np.empty_like(A_data)
    grad_B = np.empty_like(B_data)
    _fn("or_spgemm_backward", A_data.dtype)(_i64(A_rows), _p(gC), _p(C_indices), _p(C_indptr),
                                            _p(A_data), _p(A_indices), _p(A_indptr),
                                            _p(B_data), _p(B_indices), _p(B_indptr),
                                            _i64(B_data.shape[0]), _p(grad_A), _p(grad_B))
    return grad_A, grad_B


def csr_transpose(rows, cols, data, indices, indptr):
    """csr_transpose_forward_cpu, cpp/sparse_csr_cpu.cpp:311-367
    -> (At_data, At_indices, At_indptr, At_to_A_idx)."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    nnz = data.shape[0]
    At_data = np.empty_like(data)
    At_indices = np.empty(nnz, dtype=np.int64)
    At_indptr = np.empty(cols + 1, dtype=np.int64)
    At_to_A = np.empty(nnz, dtype=np.int64)
    cursor = np.empty(max(cols, 1), dtype=np.int64)
    _fn("or_csr_transpose", data.dtype)(_i64(rows), _i64(cols), _p(data), _p(indices), _p(indptr),
                                        _p(At_data), _p(At_indices), _p(At_indptr), _p(At_to_A),
                                        _p(cursor))
    return At_data, At_indices, At_indptr, At_to_A


def csr_transpose_backward(grad_At, At_to_A_idx):
    """csr_transpose_backward_cpu, cpp/sparse_csr_cpu.cpp:369-385:
    grad_A[At_to_A_idx[i]] = grad_At[i]."""
    grad_At, At_to_A_idx = _vals(grad_At), _idx(At_to_A_idx)
    grad_A = np.empty_like(grad_At)
    grad_A[At_to_A_idx] = grad_At
    return grad_A


def splincomb_forward(rows, cols, alpha, A_data, A_indices, A_indptr, beta, B_data, B_indices, B_indptr):
    """splincomb_forward_cpu, cpp/sparse_csr_cpu.cpp:387-481 -> (C_data, C_indices, C_indptr).
    alpha and beta are converted to the value type first (alpha.item<scalar_t>(), :413-414)."""
    A_data, A_indices, A_indptr = _vals(A_data), _idx(A_indices), _idx(A_indptr)
    B_data, B_indices, B_indptr = _vals(B_data, A_data.dtype), _idx(B_indices), _idx(B_indptr)
    ct = ctypes.c_float if A_data.dtype == np.float32 else ctypes.c_double
    fn = _fn("or_splincomb_forward", A_data.dtype)
    C_indptr = np.zeros(rows + 1, dtype=np.int64)
    fn(_i64(rows), ct(alpha), _p(A_data), _p(A_indices), _p(A_indptr), ct(beta), _p(B_data), _p(B_indices),
       _p(B_indptr), _p(C_indptr), None, None)
    counts = C_indptr[:rows].copy()
    C_indptr[0] = 0
    np.cumsum(counts, out=C_indptr[1:])
    nnz = int(C_indptr[rows])
    C_indices = np.empty(nnz, dtype=np.int64)
    C_data = np.empty(nnz, dtype=A_data.dtype)
    fn(_i64(rows), ct(alpha), _p(A_data), _p(A_indices), _p(A_indptr), ct(beta), _p(B_data), _p(B_indices),
       _p(B_indptr), _p(C_indptr), _p(C_indices), _p(C_data))
    return C_data, C_indices, C_indptr


def splincomb_backward(rows, cols, alpha, A_data, A_indices, A_indptr, beta, B_data, B_indices, B_indptr,
                       gC, C_indices, C_indptr):
    """splincomb_backward_cpu, cpp/sparse_csr_cpu.cpp:483-560 -> (grad_A, grad_B).  Every column of
    A and of B is present in C, so every entry of both gradients is written."""
    A_data, B_data = _vals(A_data), _vals(B_data)
    gC = _vals(gC, A_data.dtype)
    ct = ctypes.c_float if A_data.dtype == np.float32 else ctypes.c_double
    fn = _fn("or_splincomb_backward_one", A_data.dtype)
    C_indices, C_indptr = _idx(C_indices), _idx(C_indptr)
    grad_A, grad_B = np.zeros_like(A_data), np.zeros_like(B_data)
    for coef, ind, ptr, out in ((alpha, A_indices, A_indptr, grad_A), (beta, B_indices, B_indptr, grad_B)):
        ind, ptr = _idx(ind), _idx(ptr)
        fn(_i64(rows), ct(coef), _p(ind), _p(ptr), _p(gC), _p(C_indices), _p(C_indptr), _p(out))
    return grad_A, grad_B


def csr_to_dense_forward(rows, cols, data, indices, indptr):
    """csr_to_dense_forward_cpu, cpp/sparse_csr_cpu.cpp:1052-1076: zeros, then A_d[i, j] = data[k]
    in storage order (a later duplicate would overwrite an earlier one)."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    out = np.zeros((rows, cols), dtype=data.dtype)
    r = np.repeat(np.arange(rows), np.diff(indptr))
    out[r, indices] = data
    return out


def csr_to_dense_backward(grad_Ad, rows, cols, data, indices, indptr):
    """csr_to_dense_backward_cpu, cpp/sparse_csr_cpu.cpp:1078-1104: grad_A[k] = grad_Ad[i, j]."""
    indices, indptr = _idx(indices), _idx(indptr)
    r = np.repeat(np.arange(rows), np.diff(indptr))
    return np.ascontiguousarray(np.asarray(grad_Ad)[r, indices])


def csr_row_sum_forward(rows, cols, data, indices, indptr):
    """csr_row_sum_forward_cpu, cpp/sparse_csr_cpu.cpp:1106-1131."""
    data, indptr = _vals(data), _idx(indptr)
    x = np.empty(rows, dtype=data.dtype)
    _fn("or_row_sum", data.dtype)(_i64(rows), _p(data), _p(indptr), _p(x))
    return x


def csr_row_sum_backward(g, rows, cols, data, indices, indptr):
    """csr_row_sum_backward_cpu, cpp/sparse_csr_cpu.cpp:1133-1156: grad_A[k] = g[row(k)]."""
    indptr = _idx(indptr)
    return np.repeat(np.asarray(g), np.diff(indptr))


def csr_extract_diagonal_forward(rows, cols, data, indices, indptr):
    """csr_extract_diagonal_forward_cpu, cpp/sparse_csr_cpu.cpp:1158-1186."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    x = np.empty(rows, dtype=data.dtype)
    _fn("or_diagonal", data.dtype)(_i64(rows), _p(data), _p(indices), _p(indptr), _p(x))
    return x


def csr_extract_diagonal_backward(g, rows, cols, data, indices, indptr):
    """csr_extract_diagonal_backward_cpu, cpp/sparse_csr_cpu.cpp:1188-1213."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    g = _vals(g, data.dtype)
    grad_A = np.empty_like(data)
    _fn("or_diagonal_backward", data.dtype)(_i64(rows), _i64(data.shape[0]), _p(g), _p(indices), _p(indptr),
                                            _p(grad_A))
    return grad_A


def splu(rows, cols, data, indices, indptr):
    """splu_cpu, cpp/sparse_csr_cpu.cpp:777-1016 -> (M_data, M_indices, M_indptr, Mt_data, Mt_indices,
    Mt_indptr): L + U without pivoting on the filled pattern (unit diagonal of L not stored) and its
    transpose.  The matrix must be square with a stored diagonal."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    assert rows == cols
    stamp, queue = np.zeros(rows, np.int64), np.zeros(rows + 1, np.int64)
    keep = np.zeros(cols + 1, np.uint8)
    As_indptr = np.zeros(rows + 1, np.int64)
    _fn("or_splu_symbolic", data.dtype)(_i64(rows), _i64(cols), _p(indices), _p(indptr), _p(As_indptr), _p(stamp),
                                        _p(queue), _p(keep))
    nnz = int(As_indptr[rows])
    As_indices, As_data = np.empty(nnz, np.int64), np.empty(nnz, data.dtype)
    Mt_indptr, Mt_indices, Mt_data = np.empty(cols + 1, np.int64), np.empty(nnz, np.int64), np.empty(nnz, data.dtype)
    perm, cursor = np.empty(nnz, np.int64), np.empty(max(rows, cols, 1), np.int64)
    _fn("or_splu_numeric", data.dtype)(_i64(rows), _i64(cols), _p(data), _p(indices), _p(indptr), _p(As_indptr),
                                       _p(As_indices), _p(As_data), _p(Mt_indptr), _p(Mt_indices), _p(Mt_data),
                                       _p(perm), _p(stamp), _p(queue), _p(keep), _p(cursor))
    M_data, M_indices, M_indptr, _ = csr_transpose(cols, rows, Mt_data, Mt_indices, Mt_indptr)
    return M_data, M_indices, M_indptr, Mt_data, Mt_indices, Mt_indptr


def spsolve_backward(grad_x, x, rows, cols, Mt_data, Mt_indices, Mt_indptr, A_data, A_indices, A_indptr):
    """spsolve_backward_cpu, cpp/sparse_csr_cpu.cpp:1018-1048 -> (grad_A, grad_b):
    grad_b = A^-T grad_x by two solves with M^T (lower, stored diagonal; then upper, unit), and
    grad_A[k] = -(grad_b[row] * x[col])."""
    y = sptrsv_forward(rows, cols, Mt_data, Mt_indices, Mt_indptr, True, False, grad_x)
    grad_b = sptrsv_forward(rows, cols, Mt_data, Mt_indices, Mt_indptr, False, True, y)
    A_indices, A_indptr = _idx(A_indices), _idx(A_indptr)
    r = np.repeat(np.arange(rows), np.diff(A_indptr))
    x = np.asarray(x)
    grad_A = (-(grad_b[r] * x[A_indices])).astype(np.asarray(A_data).dtype)
    return grad_A, grad_b


def sptrsv_forward(rows, cols, data, indices, indptr, lower, unit, b):
    """sptrsv_forward_cpu, cpp/sparse_csr_cpu.cpp:652-723."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    b = _vals(b, data.dtype)
    x = np.empty(rows, dtype=data.dtype)
    xd = np.empty(max(rows, 1), dtype=np.float64)
    _fn("or_sptrsv_forward", data.dtype)(_i64(rows), _p(data), _p(indices), _p(indptr),
                                         ctypes.c_int(bool(lower)), ctypes.c_int(bool(unit)),
                                         _p(b), _p(x), _p(xd))
    return x


def sptrsv_backward(g, x, rows, cols, data, indices, indptr, lower, unit, b=None):
    """sptrsv_backward_cpu, cpp/sparse_csr_cpu.cpp:725-759 -> (grad_A, grad_b)."""
    data, indices, indptr = _vals(data), _idx(indices), _idx(indptr)
    g, x = _vals(g, data.dtype), _vals(x, data.dtype)
    nnz = data.shape[0]
    grad_A = np.empty_like(data)
    grad_b = np.empty(rows, dtype=data.dtype)
    At_data = np.empty_like(data)
    At_indices = np.empty(nnz, dtype=np.int64)
    At_indptr = np.empty(rows + 1, dtype=np.int64)
    At_to_A = np.empty(nnz, dtype=np.int64)
    cursor = np.empty(max(rows, 1), dtype=np.int64)
    xd = np.empty(max(rows, 1), dtype=np.float64)
    _fn("or_sptrsv_backward", data.dtype)(_i64(rows), _p(data), _p(indices), _p(indptr),
                                          ctypes.c_int(bool(lower)), ctypes.c_int(bool(unit)),
                                          _p(g), _p(x), _p(grad_A), _p(grad_b),
                                          _p(At_data), _p(At_indices), _p(At_indptr), _p(At_to_A),
                                          _p(cursor), _p(xd))
    return grad_A, grad_b
