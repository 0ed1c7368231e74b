"""Sparse CSR tensors with differentiable values on HIP devices.

Mirrors the names the reference exports from ``numml.sparse`` for the SpMV,
SpMM, SpGEMM and triangular-solve path (numml/sparse/__init__.py:1-2).
"""
from ._csr import (SparseCSRTensor, coo_to_csr, diag, eye, repack_csr, spdiag, spdmm, spgemm, spgemv,
                   splincomb, spouter, sprowsum, sptodense, sptranspose, unpack_csr)  # noqa: F401
from . import linalg  # noqa: F401
