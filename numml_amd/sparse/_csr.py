"""``SparseCSRTensor`` and the autograd Functions of the matrix-product path.

Call conventions follow the reference so that code written against
``numml.sparse`` runs on this backend unchanged:

* ``spgemv`` / ``spgemm`` / ``spdmm`` take ``(shape, data, indices, indptr, ...)``
  and return ``None`` gradients for shapes and structure
  (numml/sparse/_csr.py:102-184, 357-387);
* ``A @ x`` routes on the operand: 1-D -> SpMV, 2-D dense -> SpMM, sparse ->
  SpGEMM, N-D -> one flattened SpMM (numml/sparse/_csr.py:690-738);
* gradients live on ``A.data`` (numml/sparse/_csr.py:962-976).

The container keeps only what that path and its tests need: construction from
CSR / COO / dense / SciPy, device and dtype moves, ``to_dense`` and
``to_scipy_csr`` as checkers.
"""
import numpy as np
import torch

from .._binding import ops as _ext

__all__ = ["SparseCSRTensor", "coo_to_csr", "eye", "diag", "spgemv", "spgemm", "spdmm", "sptranspose",
           "splincomb", "sptodense", "sprowsum", "spdiag"]


def _type_error(kind_a, a, kind_b, b):
    return RuntimeError(f"{kind_a} should be same data type, got {a.type()} and {b.type()}, respectively.")


class spgemv(torch.autograd.Function):
    """y = A x with gradients for A's stored values and x (numml/sparse/_csr.py:102-133)."""

    @staticmethod
    def forward(ctx, A_shape, A_data, A_col_ind, A_rowptr, x):
        if A_data.type() != x.type():
            raise _type_error("Matrix and vector", A_data, "", x)
        y = _ext.spgemv_forward(A_shape[0], A_shape[1], A_data, A_col_ind, A_rowptr, x)
        ctx.save_for_backward(x, A_data, A_col_ind, A_rowptr)
        ctx.shape = A_shape
        return y

    @staticmethod
    def backward(ctx, grad_y):
        x, A_data, A_col_ind, A_rowptr = ctx.saved_tensors
        grad_A, grad_x = _ext.spgemv_backward(grad_y, ctx.shape[0], ctx.shape[1],
                                              A_data, A_col_ind, A_rowptr, x)
        return None, grad_A, None, None, grad_x


class spdmm(torch.autograd.Function):
    """C = A B with dense B (numml/sparse/_csr.py:357-387)."""

    @staticmethod
    def forward(ctx, A_shape, A_data, A_indices, A_indptr, B):
        if A_data.type() != B.type():
            raise _type_error("Matrices", A_data, "", B)
        if A_shape[1] != B.shape[0]:
            raise RuntimeError(
                f"Incompatible matrix shapes for multiplication.  Got {A_shape} and {B.shape}.")
        ctx.save_for_backward(A_data, A_indices, A_indptr, B)
        ctx.shape = A_shape
        return _ext.spdmm_forward(A_shape[0], A_shape[1], A_data, A_indices, A_indptr, B)

    @staticmethod
    def backward(ctx, grad_C):
        A_data, A_indices, A_indptr, B = ctx.saved_tensors
        grad_A, grad_B = _ext.spdmm_backward(ctx.shape[0], ctx.shape[1], A_data, A_indices,
                                             A_indptr, B, grad_C)
        return None, grad_A, None, None, grad_B


class spgemm(torch.autograd.Function):
    """C = A B with sparse B; returns ``(C_shape, C_data, C_indices, C_indptr)``
    (numml/sparse/_csr.py:136-184)."""

    @staticmethod
    def forward(ctx, A_shape, A_data, A_indices, A_indptr, B_shape, B_data, B_indices, B_indptr):
        if A_data.type() != B_data.type():
            raise _type_error("Matrices", A_data, "", B_data)
        if A_shape[1] != B_shape[0]:
            raise RuntimeError(
                f"Incompatible matrix shapes for multiplication.  Got {A_shape} and {B_shape}.")
        C_data, C_indices, C_indptr = _ext.spgemm_forward(
            A_shape[0], A_shape[1], A_data, A_indices, A_indptr,
            B_shape[0], B_shape[1], B_data, B_indices, B_indptr)
        ctx.save_for_backward(A_data, A_indices, A_indptr, B_data, B_indices, B_indptr,
                              C_indices, C_indptr)
        ctx.A_shape, ctx.B_shape = A_shape, B_shape
        ctx.mark_non_differentiable(C_indices, C_indptr)
        return (A_shape[0], B_shape[1]), C_data, C_indices, C_indptr

    @staticmethod
    def backward(ctx, _g_shape, grad_C_data, _g_indices, _g_indptr):
        (A_data, A_indices, A_indptr, B_data, B_indices, B_indptr,
         C_indices, C_indptr) = ctx.saved_tensors
        grad_A, grad_B = _ext.spgemm_backward(
            grad_C_data, C_indices, C_indptr,
            ctx.A_shape[0], ctx.A_shape[1], A_data, A_indices, A_indptr,
            ctx.B_shape[0], ctx.B_shape[1], B_data, B_indices, B_indptr)
        return None, grad_A, None, None, None, grad_B, None, None


class sptranspose(torch.autograd.Function):
    """A^T as a new CSR triple; returns ``(At_shape, At_data, At_indices, At_indptr)``.
    The gradient of At's values goes back through the saved permutation
    (numml/sparse/_csr.py:333-354)."""

    @staticmethod
    def forward(ctx, A_shape, A_data, A_indices, A_indptr):
        At_data, At_indices, At_indptr, At_to_A_idx = _ext.csr_transpose_forward(
            A_shape[0], A_shape[1], A_data, A_indices, A_indptr)
        ctx.save_for_backward(At_to_A_idx)
        ctx.mark_non_differentiable(At_indices, At_indptr)
        return tuple(A_shape[::-1]), At_data, At_indices, At_indptr

    @staticmethod
    def backward(ctx, _g_shape, grad_At_data, _g_indices, _g_indptr):
        (At_to_A_idx,) = ctx.saved_tensors
        return None, _ext.csr_transpose_backward(grad_At_data, At_to_A_idx), None, None


class splincomb(torch.autograd.Function):
    """C = alpha A + beta B; returns ``(C_data, C_indices, C_indptr)``.  The scalars
    get sum(A.data) and sum(B.data) as their gradients, as in the reference
    (numml/sparse/_csr.py:187-231)."""

    @staticmethod
    def forward(ctx, shape, alpha, A_data, A_col_ind, A_rowptr, beta, B_data, B_col_ind, B_rowptr):
        if A_data.type() != B_data.type():
            raise _type_error("Matrices", A_data, "", B_data)
        C_data, C_col_ind, C_rowptr = _ext.splincomb_forward(
            shape[0], shape[1], alpha, A_data, A_col_ind, A_rowptr, beta, B_data, B_col_ind, B_rowptr)
        ctx.save_for_backward(alpha, A_data, A_col_ind, A_rowptr, beta, B_data, B_col_ind, B_rowptr,
                              C_col_ind, C_rowptr)
        ctx.shape = shape
        ctx.mark_non_differentiable(C_col_ind, C_rowptr)
        return C_data, C_col_ind, C_rowptr

    @staticmethod
    def backward(ctx, grad_C_data, _g_col_ind, _g_rowptr):
        (alpha, A_data, A_col_ind, A_rowptr, beta, B_data, B_col_ind, B_rowptr,
         C_col_ind, C_rowptr) = ctx.saved_tensors
        grad_A, grad_B = _ext.splincomb_backward(
            ctx.shape[0], ctx.shape[1], alpha, A_data, A_col_ind, A_rowptr, beta, B_data, B_col_ind, B_rowptr,
            grad_C_data, C_col_ind, C_rowptr)
        return (None, torch.sum(A_data).to(alpha.device), grad_A, None, None,
                torch.sum(B_data).to(beta.device), grad_B, None, None)


def _reduction(forward_name, backward_name, doc):
    """Function of ``(A_shape, A_data, A_indices, A_indptr)`` returning one dense tensor."""

    class _Fn(torch.autograd.Function):
        @staticmethod
        def forward(ctx, A_shape, A_data, A_indices, A_indptr):
            ctx.save_for_backward(A_data, A_indices, A_indptr)
            ctx.A_shape = A_shape
            return getattr(_ext, forward_name)(A_shape[0], A_shape[1], A_data, A_indices, A_indptr)

        @staticmethod
        def backward(ctx, grad):
            A_data, A_indices, A_indptr = ctx.saved_tensors
            grad_A = getattr(_ext, backward_name)(grad, ctx.A_shape[0], ctx.A_shape[1], A_data, A_indices,
                                                  A_indptr)
            return None, grad_A, None, None

    _Fn.__doc__ = doc
    return _Fn


sptodense = _reduction("csr_to_dense_forward", "csr_to_dense_backward",
                       "Dense copy of a CSR matrix (numml/sparse/_csr.py:390-413).")
sptodense.__name__ = sptodense.__qualname__ = "sptodense"
sprowsum = _reduction("csr_row_sum_forward", "csr_row_sum_backward",
                      "Row sums of a CSR matrix (numml/sparse/_csr.py:416-438).")
sprowsum.__name__ = sprowsum.__qualname__ = "sprowsum"
spdiag = _reduction("csr_extract_diagonal_forward", "csr_extract_diagonal_backward",
                    "Diagonal of a CSR matrix (numml/sparse/_csr.py:441-463).")
spdiag.__name__ = spdiag.__qualname__ = "spdiag"


def coo_to_csr(values, row_ind, col_ind, shape, sort=True):
    """COO -> CSR.  Entries are ordered by column then (stably) by row; duplicate
    coordinates are kept as separate entries, as in numml/sparse/_csr.py:78-99."""
    if sort:
        order = torch.argsort(col_ind)
        values, row_ind, col_ind = values[order], row_ind[order], col_ind[order]
        order = torch.argsort(row_ind, stable=True)
        values, row_ind, col_ind = values[order], row_ind[order], col_ind[order]
    counts = torch.bincount(row_ind, minlength=shape[0])
    indptr = torch.zeros(shape[0] + 1, dtype=torch.int64, device=values.device)
    indptr[1:] = torch.cumsum(counts, 0)
    return values, col_ind.long(), indptr


def _unsqueeze_like(y, x):
    """Give y the singleton dimensions x has (numml/utils.py:152-167)."""
    for dim, size in enumerate(x.shape):
        if size == 1:
            y = torch.unsqueeze(y, dim)
    return y


class SparseCSRTensor(object):
    """CSR matrix whose stored values carry gradients (numml/sparse/_csr.py:549-650).

    ``SparseCSRTensor((data, indices, indptr), shape)``, ``SparseCSRTensor((data,
    (rows, cols)), shape)``, ``SparseCSRTensor(dense)`` and
    ``SparseCSRTensor(scipy_matrix)`` are accepted; ``clone=False`` adopts the
    given tensors instead of copying them.
    """

    def __init__(self, arg1, shape=None, clone=True, dtype=None, device=None):
        if isinstance(arg1, torch.Tensor):
            if arg1.layout == torch.sparse_coo:
                arg1 = arg1.coalesce()
                r, c = arg1.indices()
                self.data, self.indices, self.indptr = coo_to_csr(arg1.values(), r, c, arg1.shape)
            else:
                r, c = torch.nonzero(arg1).T
                self.data, self.indices, self.indptr = coo_to_csr(arg1[r, c], r, c, arg1.shape)
            self.shape = tuple(shape) if shape is not None else tuple(arg1.shape)
        elif isinstance(arg1, tuple) and len(arg1) == 3:
            if shape is None:
                raise RuntimeError("shape is required with (data, indices, indptr)")
            parts = []
            for i, a in enumerate(arg1):
                if isinstance(a, np.ndarray):
                    a = torch.from_numpy(np.ascontiguousarray(a))
                    a = a.clone() if clone else a
                elif clone:
                    a = torch.clone(a)
                parts.append(a)
            data, indices, indptr = parts
            if dtype is not None:
                data = data.type(dtype)
            if device is None:
                device = data.device
            self.data = data.to(device)
            self.indices = indices.long().to(device)
            self.indptr = indptr.long().to(device)
            self.shape = tuple(shape)
        elif isinstance(arg1, tuple) and len(arg1) == 2:
            if shape is None:
                raise RuntimeError("shape is required with (data, (rows, cols))")
            data, (r, c) = arg1
            self.data, self.indices, self.indptr = coo_to_csr(data, r, c, shape)
            self.shape = tuple(shape)
        elif hasattr(arg1, "tocsr"):
            m = arg1.tocsr()
            m.sort_indices()
            data = torch.from_numpy(m.data.copy())
            if dtype is not None:
                data = data.type(dtype)
            device = torch.device("cpu") if device is None else device
            self.data = data.to(device)
            self.indices = torch.from_numpy(m.indices.astype(np.int64)).to(device)
            self.indptr = torch.from_numpy(m.indptr.astype(np.int64)).to(device)
            self.shape = tuple(m.shape)
        else:
            raise RuntimeError(f"Unknown type given as argument of SparseCSRTensor: {type(arg1)}")

    # ---- products -----------------------------------------------------------
    def spmv(self, x):
        if self.shape[1] != torch.numel(x):
            raise RuntimeError("Number of columns of tensor must equal number of rows of vector.  "
                               f"Got shapes: {self.shape} and {x.shape}")
        y = spgemv.apply(self.shape, self.data, self.indices, self.indptr, x.squeeze())
        return _unsqueeze_like(y, x)

    def spdmm(self, othr):
        return spdmm.apply(self.shape, self.data, self.indices, self.indptr, othr)

    def spspmm(self, othr):
        C_shape, C_data, C_indices, C_indptr = spgemm.apply(
            self.shape, self.data, self.indices, self.indptr,
            othr.shape, othr.data, othr.indices, othr.indptr)
        # The reference re-wraps with clone=True (numml/sparse/_csr.py:685); the three tensors are
        # fresh outputs of the product, so they are adopted as they are (no copy of C).
        return SparseCSRTensor((C_data, C_indices, C_indptr), C_shape, clone=False)

    def solve_triangular(self, upper, unit, b):
        from . import linalg
        return linalg.sptrsv.apply(self.shape, self.data, self.indices, self.indptr,
                                   not upper, unit, b)

    def __matmul__(self, x):
        if isinstance(x, SparseCSRTensor):
            return self.spspmm(x)
        if not isinstance(x, torch.Tensor):
            raise RuntimeError(f"Unknown type for matmul: {type(x)}.")
        if x.ndim == 0:
            if self.shape == (1, 1):
                return self.data * x.item()
            if 1 in self.shape:
                return self.to_dense() * x.item()
            return self * x.item()
        if x.ndim == 1:
            return self.spmv(x)
        if x.ndim == 2:
            return self.spdmm(x)
        if x.shape[-2] == self.shape[1]:
            # (a_1, ..., a_k, n, b): bring n to the front, flatten the rest, one SpMM, undo
            xt = torch.transpose(x, 0, x.ndim - 2)
            y = self.spdmm(torch.flatten(xt, 1))
            return torch.transpose(y.reshape((self.shape[0],) + tuple(xt.shape[1:])), 0, x.ndim - 2)
        if 1 in x.shape:
            return self.__matmul__(torch.squeeze(x))
        raise RuntimeError(f"invalid tensor found for sparse multiply: mode {x.ndim} tensor found.  "
                           f"Trying to multiply {self.shape} sparse matrix by {x.shape} tensor.")

    def transpose(self):
        """A^T, computed eagerly as a new CSR matrix (numml/sparse/_csr.py:1074-1087)."""
        At_shape, At_data, At_indices, At_indptr = sptranspose.apply(
            self.shape, self.data, self.indices, self.indptr)
        return SparseCSRTensor((At_data, At_indices, At_indptr), At_shape, clone=False)

    def hermitian(self):
        At_shape, At_data, At_indices, At_indptr = sptranspose.apply(
            self.shape, self.data.conj(), self.indices, self.indptr)
        return SparseCSRTensor((At_data, At_indices, At_indptr), At_shape, clone=False)

    @property
    def T(self):
        return self.transpose()

    @property
    def H(self):
        return self.hermitian()

    # ---- entrywise arithmetic (numml/sparse/_csr.py:840-932) ---------------------
    @staticmethod
    def _isscalar(x):
        return isinstance(x, (int, float)) or (isinstance(x, torch.Tensor) and x.ndim == 0)

    def _lincomb(self, othr, beta, what):
        if self.shape != othr.shape:
            raise RuntimeError(f"Incompatible shapes for entrywise {what}, got {self.shape} and "
                               f"{othr.shape}, respectively.")
        C = splincomb.apply(self.shape, torch.tensor(1.), self.data, self.indices, self.indptr,
                            torch.tensor(beta), othr.data, othr.indices, othr.indptr)
        return SparseCSRTensor(C, self.shape, clone=False)

    def __add__(self, othr):
        if SparseCSRTensor._isscalar(othr):
            return SparseCSRTensor((self.data + othr, self.indices, self.indptr), self.shape, clone=False)
        if isinstance(othr, SparseCSRTensor):
            return self._lincomb(othr, 1., "addition")
        raise RuntimeError(f"Unknown type for sparse tensor addition: {type(othr)}.")

    def __sub__(self, othr):
        if SparseCSRTensor._isscalar(othr):
            # the reference adds the scalar here as well (numml/sparse/_csr.py:898-899)
            return SparseCSRTensor((self.data + othr, self.indices, self.indptr), self.shape, clone=False)
        if isinstance(othr, SparseCSRTensor):
            return self._lincomb(othr, -1., "subtraction")
        raise RuntimeError(f"Unknown type for sparse tensor addition: {type(othr)}.")

    def __mul__(self, s):
        if SparseCSRTensor._isscalar(s):
            return SparseCSRTensor((self.data * s, self.indices, self.indptr), self.shape, clone=False)
        if isinstance(s, torch.Tensor) and len(torch.squeeze(s).shape) == 2:
            raise RuntimeError("Element-wise hadamard product not implemented")
        raise RuntimeError(f"Unknown type for multiplication: {type(s)}.")

    __rmul__ = __mul__

    def __rtruediv__(self, other):
        if SparseCSRTensor._isscalar(other):
            return SparseCSRTensor((other / self.data, self.indices, self.indptr), self.shape, clone=False)
        raise RuntimeError(f"Unknown type for right-division: {type(other)}.")

    def __neg__(self):
        return SparseCSRTensor((-self.data, self.indices, self.indptr), self.shape, clone=False)

    def __pow__(self, p):
        return SparseCSRTensor((self.data ** p, self.indices, self.indptr), self.shape, clone=False)

    def abs(self):
        return SparseCSRTensor((torch.abs(self.data), self.indices, self.indptr), self.shape, clone=False)

    __abs__ = abs

    # ---- reductions ----------------------------------------------------------------
    def sum(self):
        return self.data.sum()

    def row_sum(self):
        """x[i] = sum of the stored entries of row i (numml/sparse/_csr.py:852-861)."""
        return sprowsum.apply(self.shape, self.data, self.indices, self.indptr)

    def diagonal(self):
        """Stored diagonal entries, 0 where a row has none (numml/sparse/_csr.py:1016-1027)."""
        return spdiag.apply(self.shape, self.data, self.indices, self.indptr)

    def trace(self):
        return self.diagonal().sum()

    # ---- conversions ----------------------------------------------------------
    @property
    def row_indices(self):
        """Row of every stored entry (numml/sparse/_csr.py:1002-1014)."""
        counts = self.indptr[1:] - self.indptr[:-1]
        return torch.repeat_interleave(
            torch.arange(self.shape[0], device=self.indptr.device), counts)

    @property
    def diagonal_idx(self):
        """Position of the stored diagonal entry of each row, -1 where a row has none
        (numml/sparse/_csr.py:985-1000)."""
        n = min(self.shape)
        idx = torch.full((n,), -1, dtype=torch.int64, device=self.indices.device)
        rows = self.row_indices
        hit = (self.indices == rows) & (rows < n)
        idx[rows[hit]] = torch.nonzero(hit).flatten()
        return idx

    def _band(self, keep):
        rows = self.row_indices
        counts = torch.bincount(rows[keep], minlength=self.shape[0])
        indptr = torch.zeros(self.shape[0] + 1, dtype=torch.int64, device=self.indptr.device)
        indptr[1:] = torch.cumsum(counts, 0)
        # indexing keeps the gradient path to the selected entries; the others get zero
        return SparseCSRTensor((self.data[keep], self.indices[keep], indptr), self.shape)

    def tril(self, k=0):
        """Entries with column <= row + k (numml/sparse/_csr.py:234-280, 1063-1065)."""
        return self._band(self.indices <= self.row_indices + k)

    def triu(self, k=0):
        """Entries with column >= row + k (numml/sparse/_csr.py:283-330, 1067-1069)."""
        return self._band(self.indices >= self.row_indices + k)

    def to_dense(self):
        """Dense copy; gradients flow to and from the stored entries
        (numml/sparse/_csr.py:740-751)."""
        return sptodense.apply(self.shape, self.data, self.indices, self.indptr)

    def to_coo(self):
        """torch's sparse COO tensor of the stored entries; gradients on the values carry over
        (numml/sparse/_csr.py:753-769)."""
        return torch.sparse_coo_tensor(torch.stack((self.row_indices, self.indices)), self.data, self.shape,
                                       device=self.device)

    def tocoo(self):
        """SciPy COO matrix (numml/sparse/_csr.py:771-788); gradient information is dropped."""
        import scipy.sparse as sp
        return sp.coo_matrix((self.data.detach().cpu().numpy(),
                              (self.row_indices.cpu().numpy().astype("int32"),
                               self.indices.cpu().numpy().astype("int32"))), shape=self.shape)

    def to_scipy_csr(self):
        import scipy.sparse as sp
        return sp.csr_matrix((self.data.detach().cpu().numpy(), self.indices.cpu().numpy(),
                              self.indptr.cpu().numpy()), shape=self.shape)

    tocsr = to_scipy_csr

    def conjugate(self):
        """Element-wise complex conjugation (numml/sparse/_csr.py:1041-1061)."""
        return SparseCSRTensor((torch.clone(self.data.conj()), self.indices, self.indptr), self.shape, clone=False)

    conj = conjugate

    def to(self, device):
        return SparseCSRTensor((self.data.to(device), self.indices.to(device),
                                self.indptr.to(device)), self.shape, clone=False)

    def cpu(self):
        return self.to(torch.device("cpu"))

    def cuda(self, device=None):
        return self.to(torch.device("cuda", torch.cuda.current_device() if device is None else device))

    def type(self, dtype):
        return SparseCSRTensor((self.data.type(dtype), self.indices, self.indptr), self.shape,
                               clone=False)

    def double(self):
        return self.type(torch.float64)

    def float(self):
        return self.type(torch.float32)

    def detach(self):
        return SparseCSRTensor((self.data.detach(), self.indices, self.indptr), self.shape,
                               clone=False)

    def clone(self):
        return SparseCSRTensor((self.data, self.indices, self.indptr), self.shape)

    copy = clone

    # ---- properties -------------------------------------------------------------
    @property
    def requires_grad(self):
        return self.data.requires_grad

    @requires_grad.setter
    def requires_grad(self, flag):
        self.data.requires_grad = flag

    @property
    def grad(self):
        # a copy of the values, as in the reference (numml/sparse/_csr.py:620-637 clones what it
        # wraps): editing A.grad in place must not change the gradient autograd accumulates into.
        # The pattern tensors are shared with A.
        return SparseCSRTensor((self.data.grad.clone(), self.indices, self.indptr), self.shape, clone=False)

    @property
    def grad_fn(self):
        return self.data.grad_fn

    @property
    def nnz(self):
        return len(self.data)

    @property
    def device(self):
        return self.data.device

    @property
    def dtype(self):
        return self.data.dtype

    def __repr__(self):
        extra = "" if self.device.type == "cpu" else f", device='{self.device}'"
        extra += ", requires_grad=True" if self.requires_grad else ""
        return (f"<{self.shape[0]}x{self.shape[1]} sparse matrix tensor of type '{self.data.dtype}'\n"
                f"\twith {self.nnz} stored elements in Compressed Sparse Row format{extra}>")


def eye(N, k=0, dtype=torch.float32, device=None):
    """Ones on the k-th diagonal of an N x N matrix (numml/sparse/_csr.py:467-486)."""
    if abs(k) >= N:
        raise RuntimeError("Specified bandwidth for eye() is larger than matrix size.  "
                           f"Got k={abs(k)}, N={N}.")
    n = max(N - abs(k), 0)
    rows = torch.arange(n, dtype=torch.int64) + max(-k, 0)
    cols = rows + k
    counts = torch.zeros(N, dtype=torch.int64)
    counts[rows] = 1
    indptr = torch.zeros(N + 1, dtype=torch.int64)
    indptr[1:] = torch.cumsum(counts, 0)
    out = SparseCSRTensor((torch.ones(n, dtype=dtype), cols, indptr), (N, N), clone=False)
    return out if device is None else out.to(device)


def spouter(x, y):
    """x y^T on the pattern of the nonzeros of x times the nonzeros of y
    (numml/sparse/_csr.py:511-538)."""
    x_nz = torch.nonzero(x).flatten()
    y_nz = torch.nonzero(y).flatten()
    row, col = torch.meshgrid(x_nz, y_nz, indexing="ij")
    row, col = row.flatten(), col.flatten()
    return SparseCSRTensor((x[row] * y[col], (row, col)), shape=(len(x), len(y)))


def unpack_csr(A):
    return A.data, A.indices, A.indptr, A.shape


def repack_csr(A_data, A_indices, A_indptr, A_shape):
    return SparseCSRTensor((A_data, A_indices, A_indptr), A_shape, clone=False)


def diag(x, k=0):
    """Square matrix with the vector x on its k-th diagonal (numml/sparse/_csr.py:489-508);
    gradients flow back to x through the stored values."""
    n = len(x)
    N = n + abs(k)
    rows = torch.arange(n, dtype=torch.int64, device=x.device) + max(-k, 0)
    return SparseCSRTensor((x, (rows, rows + k)), shape=(N, N))
