"""CPU-only checks of the boundary: the library exports what include/numml_hip.h
declares, the Python mirror keeps the reference's names and error behaviour, and
the host-side container logic (COO -> CSR, shapes, dtype moves) works.  No compute
entry point is called here (there is no GPU)."""
import ctypes
import inspect
import os
import re

import numpy as np
import pytest
import torch

import numml_amd
from numml_amd import _lib, numml_torch_cpp as ext, sparse as sp
from numml_amd.sparse import linalg

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "numml_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nm_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert len(names) >= 20
    L = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, f"declared in numml_hip.h but not exported: {missing}"


def test_ctypes_table_covers_the_header():
    L = _lib.lib()
    table = set(_lib._SIGNATURES) | {"nm_version", "nm_last_error", "nm_sptrsv_plan_levels",
                                     "nm_sptrsv_plan_launches", "nm_sptrsv_plan_chain_levels",
                                     "nm_sptrsv_plan_shared_launches", "nm_sptrsv_plan_destroy"}
    assert set(_declared()) == table
    assert L.nm_version() == 1001
    assert L.nm_last_error() == b""


def test_argument_checks_report_through_nm_last_error():
    L = _lib.lib()
    nbytes = ctypes.c_size_t(0)
    assert L.nm_spgemm_workspace_bytes(-1, 5, ctypes.byref(nbytes)) == 1            # NM_ERR_INVALID
    assert b"negative" in L.nm_last_error()
    assert L.nm_spgemm_workspace_bytes(2 ** 31, 5, ctypes.byref(nbytes)) == 4       # NM_ERR_UNSUPPORTED
    assert L.nm_spgemm_workspace_bytes(1000, 1000, ctypes.byref(nbytes)) == 0 and nbytes.value > 0
    with pytest.raises(_lib.NummlHipError, match="status 1"):
        _lib.check(L.nm_spgemv_forward(7, 1, 1, 1, None, None, None, None, None, None), "nm_spgemv_forward")
    # product plans: a class nm_spgemm_plan_build never reports, a plan memory that is too small, and
    # sizes beyond what a plan's 32-bit positions hold -- all refused on the host, nothing launched
    assert L.nm_spgemm_numeric_planned(1, 0, 4, 4, 4, 4, None, None, None, None, None, None, None) == 1
    assert b"plan class" in L.nm_last_error()
    pbytes = ctypes.c_size_t(0)
    assert L.nm_spgemm_plan_bytes(1000, ctypes.byref(pbytes)) == 0 and pbytes.value >= 28 * 1000
    usable = ctypes.c_int(7)
    assert L.nm_spgemm_plan_adopt(4, 4, 1000, 10, 10, 0, ctypes.c_void_p(8), ctypes.c_void_p(8), 16, None,
                                  ctypes.byref(usable), None) == 3                  # NM_ERR_WORKSPACE
    assert L.nm_spgemm_plan_adopt(4, 4, 2 ** 31, 10, 10, 0, ctypes.c_void_p(8), ctypes.c_void_p(8), 2 ** 40, None,
                                  ctypes.byref(usable), None) == 0 and usable.value == 0
    assert L.nm_spgemm_plan_adopt(4, 4, 1000, 10, 10, 5, ctypes.c_void_p(8), ctypes.c_void_p(8), 2 ** 40, None,
                                  ctypes.byref(usable), None) == 0 and usable.value == 0    # rows on the hash path


def test_mirror_has_the_reference_signatures():
    # cpp/sparse_csr.hpp:32-105
    want = {
        "spgemv_forward": ["A_rows", "A_cols", "A_data", "A_col_ind", "A_rowptr", "x"],
        "spgemv_backward": ["grad_z", "A_rows", "A_cols", "A_data", "A_col_ind", "A_rowptr", "x"],
        "spgemm_forward": ["A_rows", "A_cols", "A_data", "A_indices", "A_indptr",
                           "B_rows", "B_cols", "B_data", "B_indices", "B_indptr"],
        "spgemm_backward": ["grad_C", "C_indices", "C_indptr", "A_rows", "A_cols", "A_data", "A_indices",
                            "A_indptr", "B_rows", "B_cols", "B_data", "B_indices", "B_indptr"],
        "spdmm_forward": ["A_rows", "A_cols", "A_data", "A_indices", "A_indptr", "B"],
        "spdmm_backward": ["A_rows", "A_cols", "A_data", "A_indices", "A_indptr", "B", "grad_C"],
        "sptrsv_forward": ["A_rows", "A_cols", "A_data", "A_indices", "A_indptr", "lower", "unit", "b"],
        "sptrsv_backward": ["grad_x", "x", "A_rows", "A_cols", "A_data", "A_indices", "A_indptr",
                            "lower", "unit", "b"],
        "splu": ["A_rows", "A_cols", "A_data", "A_indices", "A_indptr"],                   # :107-111
        "spsolve_backward": ["grad_x", "x", "A_rows", "A_cols", "Mt_data", "Mt_indices", "Mt_indptr",
                             "A_data", "A_indices", "A_indptr"],                            # :113-118
    }
    for name, params in want.items():
        assert list(inspect.signature(getattr(ext, name)).parameters) == params, name


def test_cpu_tensors_are_refused_not_computed():
    d, i, p = torch.ones(3), torch.tensor([0, 1, 2]), torch.tensor([0, 1, 2, 3])
    x = torch.ones(3)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        ext.spgemv_forward(3, 3, d, i, p, x)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        ext.spdmm_forward(3, 3, d, i, p, torch.ones(3, 2))
    with pytest.raises(RuntimeError, match="HIP devices only"):
        ext.spgemm_forward(3, 3, d, i, p, 3, 3, d, i, p)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        ext.sptrsv_forward(3, 3, d, i, p, True, False, x)
    A = sp.SparseCSRTensor((d, i, p), (3, 3))
    with pytest.raises(RuntimeError, match="HIP devices only"):
        A @ x


def test_compiled_extension_exports_the_reference_module():
    import numml_amd
    cpp = numml_amd.load_compiled()
    names = [f"{op}_{d}" for op in ("spgemv", "spgemm", "csr_transpose", "splincomb", "spdmm", "sptrsv",
                                    "csr_to_dense", "csr_row_sum", "csr_extract_diagonal")
             for d in ("forward", "backward")] + ["splu", "spsolve_backward"]      # cpp/sparse_csr.cpp:307-319
    assert len(names) == 20
    for name in names:
        assert callable(getattr(cpp, name)), name
        assert callable(getattr(ext, name)), name
    d, i, p = torch.ones(3), torch.tensor([0, 1, 2]), torch.tensor([0, 1, 2, 3])
    with pytest.raises(RuntimeError, match="HIP devices only"):
        cpp.spgemv_forward(3, 3, d, i, p, torch.ones(3))
    with pytest.raises(RuntimeError, match="HIP devices only"):
        cpp.spgemm_forward(3, 3, d, i, p, 3, 3, d, i, p)
    with pytest.raises(RuntimeError, match="HIP devices only"):
        cpp.sptrsv_backward(d, d, 3, 3, d, i, p, True, False, d)
    assert cpp.backward_mode() in ("planned", "eager", "atomic") and cpp.plan_cache_size() == 0


def test_function_level_errors_match_the_reference():
    d, i, p = torch.ones(3), torch.tensor([0, 1, 2]), torch.tensor([0, 1, 2, 3])
    A = sp.SparseCSRTensor((d, i, p), (3, 3))
    with pytest.raises(RuntimeError, match="same data type"):       # numml/sparse/_csr.py:109-110
        A @ torch.ones(3, dtype=torch.float64)
    with pytest.raises(RuntimeError, match="Number of columns"):     # :653-654
        A @ torch.ones(4)
    with pytest.raises(RuntimeError, match="Incompatible matrix shapes"):   # :365-366
        A @ torch.ones(4, 2)
    with pytest.raises(RuntimeError, match="Incompatible matrix shapes"):   # :148-149
        A @ sp.SparseCSRTensor((torch.ones(1), torch.tensor([0]), torch.tensor([0, 1, 1])), (2, 3))
    R = sp.SparseCSRTensor((torch.ones(1), torch.tensor([0]), torch.tensor([0, 1, 1])), (2, 3))
    with pytest.raises(RuntimeError, match="Expected square matrix"):       # numml/sparse/linalg.py:15-16
        linalg.spsolve_triangular(R, torch.ones(2))
    with pytest.raises(RuntimeError, match="Unknown type for matmul"):
        A @ 3


def test_coo_to_csr_orders_by_row_then_column_and_keeps_duplicates():
    vals = torch.tensor([1., 2., 3., 4., 5.])
    rows = torch.tensor([2, 0, 2, 0, 2])
    cols = torch.tensor([1, 3, 0, 1, 1])
    A = sp.SparseCSRTensor((vals, (rows, cols)), shape=(3, 4))
    assert A.indptr.tolist() == [0, 2, 2, 5]
    assert A.indices.tolist() == [1, 3, 0, 1, 1]
    assert A.data[:3].tolist() == [4., 2., 3.] and sorted(A.data[3:].tolist()) == [1., 5.]   # duplicates kept
    assert A.nnz == 5 and A.shape == (3, 4)


def test_container_from_dense_scipy_and_moves():
    import scipy.sparse as sps
    D = torch.tensor([[0., 2., 0.], [1., 0., 3.]])
    A = sp.SparseCSRTensor(D)
    assert A.indptr.tolist() == [0, 1, 3] and A.indices.tolist() == [1, 0, 2] and A.data.tolist() == [2., 1., 3.]
    assert np.array_equal(A.to_scipy_csr().toarray(), D.numpy())
    with pytest.raises(RuntimeError, match="HIP devices only"):      # to_dense is a device op, like the products
        A.to_dense()
    S = sp.SparseCSRTensor(sps.random(20, 30, 0.2, random_state=1, format="coo"))
    assert S.shape == (20, 30) and S.indices.dtype == torch.int64 and S.data.dtype == torch.float64
    assert S.to_scipy_csr().nnz == S.nnz
    assert S.float().dtype == torch.float32 and S.double().dtype == torch.float64
    C = A.clone()
    C.data[0] = 9.0
    assert A.data[0] == 2.0
    A.requires_grad = True
    assert A.requires_grad and A.data.requires_grad
    (A.data * torch.tensor([2., 4., 6.])).sum().backward()           # gradients live on A.data
    assert A.grad.data.tolist() == [2., 4., 6.]
    # A.grad wraps a COPY of the values, like the reference's constructor (numml/sparse/_csr.py:620-637):
    # an in-place edit of it leaves the gradient autograd accumulates into alone
    A.grad.data.zero_()
    assert A.data.grad.tolist() == [2., 4., 6.]
    assert A.grad.indices.data_ptr() == A.indices.data_ptr()          # the pattern is shared
    E = sp.eye(4, k=-1)
    assert E.indptr.tolist() == [0, 0, 1, 2, 3] and E.indices.tolist() == [0, 1, 2]
    assert "sparse matrix tensor" in repr(A)


def test_product_path_does_not_touch_the_oracle():
    # the oracle is test infrastructure: nothing under numml_amd/ may import it
    pkg = os.path.dirname(numml_amd.__file__)
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f
                assert "liboracle" not in text, f


def test_integration_snippet_runs():
    # the integration guide's "keep the reference's CPU path" block, executed as written against a
    # stand-in for the reference's compiled module
    import sys
    import types
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = re.search(r"```python\n(import numml_torch_cpp as ref_ext.*?)```", text, flags=re.S).group(1)
    stub = types.ModuleType("numml_torch_cpp")
    calls = []
    for name in ("spgemv", "spdmm", "spgemm", "sptrsv"):
        for d in ("forward", "backward"):
            setattr(stub, f"{name}_{d}", lambda *a, _n=f"{name}_{d}": calls.append(_n) or "cpu")
    saved = sys.modules.get("numml_torch_cpp")
    sys.modules["numml_torch_cpp"] = stub
    try:
        exec(compile(block, "INTEGRATION.md", "exec"), {})
        d, i, p = torch.ones(3), torch.tensor([0, 1, 2]), torch.tensor([0, 1, 2, 3])
        assert stub.spgemv_forward(3, 3, d, i, p, torch.ones(3)) == "cpu"      # CPU tensors -> the reference
        assert stub.sptrsv_forward(3, 3, d, i, p, True, False, torch.ones(3)) == "cpu"
        assert calls == ["spgemv_forward", "sptrsv_forward"]
    finally:
        if saved is None:
            del sys.modules["numml_torch_cpp"]
        else:
            sys.modules["numml_torch_cpp"] = saved


@pytest.mark.parametrize("binding", ["ctypes", "compiled"])
def test_mismatched_sizes_raise_before_anything_is_launched(binding):
    # every length a kernel would index with is checked on the host; CPU tensors suffice to see it,
    # because the shape checks come before the device check
    m = ext if binding == "ctypes" else numml_amd.load_compiled()
    d, i, p = torch.ones(3), torch.tensor([0, 1, 2]), torch.tensor([0, 1, 2, 3])
    x, X = torch.ones(3), torch.ones(3, 2)
    bad = [
        (m.spgemv_forward, (3, 3, d, i, p[:3], x), "row pointers"),
        (m.spgemv_forward, (3, 3, d, i[:2], p, x), "equal length"),
        (m.spgemv_forward, (3, 3, d, i, p, torch.ones(4)), "x with 3 entries"),
        (m.spgemv_forward, (3, 4, d, i, p, x), "x with 4 entries"),
        (m.spgemv_backward, (torch.ones(2), 3, 3, d, i, p, x), "grad_z with 3 entries"),
        (m.spdmm_forward, (3, 3, d, i, p, torch.ones(4, 2)), "B of shape 3 x n"),
        (m.spdmm_backward, (3, 3, d, i, p, X, torch.ones(3, 3)), "grad_C of shape 3 x 2"),
        (m.spgemm_forward, (3, 3, d, i, p, 4, 3, d, i, torch.tensor([0, 1, 2, 3, 3])), "columns but B has"),
        (m.spgemm_forward, (3, 3, d, i, p, 3, 3, d, i, p[:2]), "row pointers"),
        (m.spgemm_backward, (torch.ones(2), i, p, 3, 3, d, i, p, 3, 3, d, i, p), "equal length"),
        (m.sptrsv_forward, (3, 3, d, i, p, True, False, torch.ones(2)), "b with 3 entries"),
        (m.sptrsv_forward, (3, 4, d, i, p, True, False, x), "square"),
        (m.sptrsv_backward, (x, torch.ones(5), 3, 3, d, i, p, True, False, x), "x with 3 entries"),
        (m.csr_transpose_forward, (3, 3, d, i, p[:1]), "row pointers"),
        (m.csr_transpose_backward, (d, i[:2]), "At_to_A_idx with 3 entries"),
        (m.splincomb_forward, (3, 3, torch.tensor(1.0), d, i, p, torch.tensor(1.0), d, i, p[:3]), "row pointers"),
        (m.csr_to_dense_forward, (2, 3, d, i, p), "row pointers"),
        (m.csr_row_sum_backward, (torch.ones(4), 3, 3, d, i, p), "grad_x with 3 entries"),
        (m.csr_extract_diagonal_forward, (3, 3, d[:2], i, p), "equal length"),
        (m.splu, (3, 3, d, i, p[:2]), "row pointers"),
        (m.spsolve_backward, (x, x, 3, 3, d, i, p, d, i[:1], p), "equal length"),
    ]
    for fn, args, msg in bad:
        with pytest.raises(RuntimeError, match=msg):
            fn(*args)
    # well-formed CPU tensors get past the shape checks and are refused for their device
    with pytest.raises(RuntimeError, match="HIP devices only"):
        m.spgemv_forward(3, 3, d, i, p, x)
