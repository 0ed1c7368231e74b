"""ctypes binding of libnumml_hip.so (the C ABI declared in include/numml_hip.h).

The library is the only compute path of this package: if it is missing, loading
raises; nothing falls back to the CPU.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libnumml_hip.so")

NM_F32, NM_F64 = 0, 1
NM_OK = 0

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_ptr = ctypes.c_void_p
_c_size = ctypes.c_size_t
_c_dbl = ctypes.c_double

# name -> argtypes, in the order of include/numml_hip.h
_SIGNATURES = {
    "nm_spgemv_forward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_spgemv_backward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                           _c_ptr, _c_ptr, _c_ptr],
    "nm_structure_hash_bytes": [ctypes.POINTER(_c_size)],
    "nm_structure_hash": [_c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr, ctypes.POINTER(ctypes.c_uint64),
                          _c_ptr],
    "nm_csr_transpose_plan_bytes": [_c_i64, _c_i64, _c_i64, ctypes.POINTER(_c_size), ctypes.POINTER(_c_size)],
    "nm_csr_transpose_plan_build": [_c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr, _c_size,
                                    _c_ptr],
    "nm_csr_longest_row": [_c_i64, _c_ptr, _c_ptr, _c_size, _c_ptr, ctypes.POINTER(_c_i64), _c_ptr],
    "nm_csr_transpose_plan_info": [_c_i64, _c_i64, _c_i64, _c_ptr, ctypes.POINTER(ctypes.c_int32), _c_ptr],
    "nm_stream_probe": [_c_ptr, _c_size, _c_ptr, _c_size, _c_ptr],
    "nm_spgemv_forward_planned": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_spgemv_forward_planned_lists": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_spgemv_backward_planned": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                   _c_ptr, _c_ptr],
    "nm_spgemv_backward_planned_lists": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                   _c_ptr, _c_ptr],
    "nm_spdmm_backward_planned": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64,
                                  _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_ptr],
    "nm_spdmm_forward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64,
                         _c_ptr, _c_i64, _c_ptr],
    "nm_spdmm_backward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64,
                          _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_ptr],
    "nm_spgemm_workspace_bytes": [_c_i64, _c_i64, ctypes.POINTER(_c_size)],
    "nm_spgemm_symbolic": [_c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                           _c_size, _c_ptr, _c_ptr],
    "nm_spgemm_symbolic_result": [_c_i64, _c_i64, _c_ptr, _c_size, ctypes.POINTER(_c_i64),
                                  ctypes.POINTER(_c_i64), _c_ptr, _c_ptr],
    "nm_spgemm_numeric": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                          _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_i64, _c_ptr],
    "nm_spgemm_backward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                           _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_spgemm_backward_planned": [_c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                   _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_spgemm_symbolic_mapped": [_c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                  _c_ptr, _c_size, _c_ptr, _c_size, _c_ptr, _c_ptr],
    "nm_spgemm_numeric_mapped": [_c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                 _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_i64, _c_ptr, _c_size,
                                 _c_int, _c_ptr],
    "nm_spgemm_plan_adopt": [_c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_size, _c_ptr,
                             ctypes.POINTER(_c_int), _c_ptr],
    "nm_spgemm_plan_bytes": [_c_i64, ctypes.POINTER(_c_size)],
    "nm_spgemm_plan_build": [_c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                             _c_ptr, _c_ptr, _c_size, _c_ptr, ctypes.POINTER(_c_int), _c_ptr],
    "nm_spgemm_numeric_planned": [_c_int, _c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                  _c_ptr, _c_ptr, _c_ptr],
    "nm_spgemm_backward_mapped": [_c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                  _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_spgemm_plan_bytes_wide": [_c_i64, _c_int, ctypes.POINTER(_c_size)],
    "nm_spgemm_plan_build_wide": [_c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                  _c_ptr, _c_ptr, _c_ptr, _c_size, _c_int, _c_ptr, ctypes.POINTER(_c_int), _c_ptr],
    "nm_spgemm_backward_mapped_wide": [_c_int, _c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr,
                                       _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_sptrsv_plan_bytes": [_c_i64, _c_i64, ctypes.POINTER(_c_size), ctypes.POINTER(_c_size)],
    "nm_sptrsv_analyse": [_c_i64, _c_i64, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_size, _c_ptr, _c_size,
                          ctypes.POINTER(_c_ptr), _c_ptr],
    "nm_sptrsv_solve_bytes": [_c_i64, _c_i64, ctypes.POINTER(_c_size)],
    "nm_sptrsv_solve": [_c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr],
    "nm_sptrsv_configure": [_c_i64, _c_int],
    "nm_spgemv_configure": [_c_int],
    "nm_sptrsv_solve_static_capacity": [ctypes.POINTER(_c_size)],
    "nm_sptrsv_solve_static": [_c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr],
    "nm_csr_transpose_forward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                 _c_ptr],
    "nm_csr_transpose_backward": [_c_int, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_splincomb_workspace_bytes": [_c_i64, ctypes.POINTER(_c_size)],
    "nm_splincomb_symbolic": [_c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr],
    "nm_splincomb_numeric": [_c_int, _c_i64, _c_dbl, _c_ptr, _c_ptr, _c_ptr, _c_dbl, _c_ptr, _c_ptr, _c_ptr,
                             _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_splincomb_backward": [_c_int, _c_i64, _c_dbl, _c_ptr, _c_ptr, _c_dbl, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                              _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_splincomb_plan_bytes": [_c_i64, _c_i64, _c_i64, ctypes.POINTER(_c_size)],
    "nm_splincomb_plan_build": [_c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                _c_size, _c_ptr],
    "nm_splincomb_numeric_planned": [_c_int, _c_i64, _c_i64, _c_i64, _c_dbl, _c_ptr, _c_dbl, _c_ptr, _c_ptr, _c_ptr,
                                     _c_ptr],
    "nm_splincomb_backward_planned": [_c_int, _c_i64, _c_i64, _c_i64, _c_dbl, _c_dbl, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                      _c_ptr],
    "nm_csr_to_dense_forward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr],
    "nm_csr_to_dense_backward": [_c_int, _c_i64, _c_i64, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_csr_row_sum_forward": [_c_int, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_csr_row_sum_backward": [_c_int, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_csr_extract_diagonal_forward": [_c_int, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_csr_extract_diagonal_backward": [_c_int, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_splu_symbolic_bytes": [_c_i64, ctypes.POINTER(_c_size)],
    "nm_splu_symbolic": [_c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr],
    "nm_splu_fill": [_c_int, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_ptr],
    "nm_splu_values": [_c_int, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    "nm_splu_numeric_bytes": [_c_i64, ctypes.POINTER(_c_size)],
    "nm_splu_numeric": [_c_int, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_size, _c_i64, _c_ptr],
    "nm_masked_outer": [_c_int, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_dbl, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
}

_lib = None


class NummlHipError(RuntimeError):
    pass


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NummlHipError(
            f"{LIB_PATH} is missing: build it with `python -m numml_amd.build` "
            "(this backend has no CPU fallback)")
    L = ctypes.CDLL(LIB_PATH)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(L, name)
        fn.argtypes = argtypes
        fn.restype = _c_int
    L.nm_version.restype = _c_int
    L.nm_last_error.restype = ctypes.c_char_p
    L.nm_sptrsv_plan_levels.argtypes = [_c_ptr]
    L.nm_sptrsv_plan_levels.restype = _c_i64
    L.nm_sptrsv_plan_launches.argtypes = [_c_ptr]
    L.nm_sptrsv_plan_launches.restype = _c_i64
    L.nm_sptrsv_plan_chain_levels.argtypes = [_c_ptr, _c_int]
    L.nm_sptrsv_plan_chain_levels.restype = _c_i64
    L.nm_sptrsv_plan_shared_launches.argtypes = [_c_ptr, _c_int]
    L.nm_sptrsv_plan_shared_launches.restype = _c_i64
    L.nm_sptrsv_plan_destroy.argtypes = [_c_ptr]
    L.nm_sptrsv_plan_destroy.restype = None
    _lib = L
    return _lib


def check(status, what):
    if status != NM_OK:
        msg = lib().nm_last_error().decode("utf-8", "replace")
        raise NummlHipError(f"{what} failed with status {status}: {msg}")
