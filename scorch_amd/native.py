"""ctypes binding of libscorch_hip.so (declarations: include/scorch_hip.h and, for the single
steps this package drives itself, include/scorch_hip_unstable.h).

The library is loaded from this directory.  If it is not there it is built
once with hipcc (scorch_amd.build); if that is impossible the import of the
kernels fails with an error -- there is no fallback implementation.
"""
from __future__ import annotations

import ctypes
import os
import threading
from typing import Optional

from . import build as _build

_i64 = ctypes.c_int64
_ptr = ctypes.c_void_p
_size = ctypes.c_size_t

OK, EINVAL, EWORKSPACE, ERUNTIME, EUNSUPPORTED = 0, 1, 2, 3, 4

_SPMM = [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _size, _ptr]
_SPMM_ROWS = [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, ctypes.c_int, _ptr, _ptr]
_SPMM_PLANNED = [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, ctypes.c_int, _ptr, _ptr, _size, _ptr, _size,
                 _ptr]
_SPGEMM = [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _size, _ptr]
_SPMV = [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _size, _ptr]

# name -> (restype, argtypes); one entry per declaration in the two headers
SIGNATURES = {
    "scorch_hip_abi_version": (ctypes.c_int, []),
    "scorch_hip_last_error": (ctypes.c_char_p, []),
    "scorch_hip_init": (ctypes.c_int, []),
    "scorch_hip_csr_plan_create": (ctypes.c_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, ctypes.POINTER(_ptr)]),
    "scorch_hip_csr_plan_destroy": (ctypes.c_int, [_ptr]),
    "scorch_hip_csr_plan_info": (ctypes.c_int, [_ptr, ctypes.POINTER(_i64)]),
    "scorch_hip_csr_plan_prepare": (ctypes.c_int, [_ptr, ctypes.c_int, _i64, _ptr]),
    "scorch_hip_spmm_csr_plan_f32": (ctypes.c_int, [_ptr, _i64, _ptr, _ptr, _ptr, ctypes.c_int, _ptr, _ptr]),
    "scorch_hip_sddmm_csr_plan_f32": (ctypes.c_int, [_ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "scorch_hip_softmax_csr_plan_f32": (ctypes.c_int, [_ptr, _ptr, ctypes.c_float, _ptr, _ptr]),
    "scorch_hip_dense_plan_create": (ctypes.c_int, [_i64, _i64, _ptr, _ptr, ctypes.POINTER(_ptr)]),
    "scorch_hip_dense_plan_update": (ctypes.c_int, [_ptr, _ptr]),
    "scorch_hip_dense_plan_destroy": (ctypes.c_int, [_ptr]),
    "scorch_hip_spmm_csr_plan_dense_f32": (ctypes.c_int, [_ptr, _ptr, _ptr, _ptr, ctypes.c_int, _ptr, _ptr]),
    "scorch_hip_timing_begin": (ctypes.c_int, []),
    "scorch_hip_timing_end": (ctypes.c_int, [ctypes.POINTER(ctypes.c_float), ctypes.c_int,
                                             ctypes.POINTER(ctypes.c_int)]),
    "scorch_hip_spmm_csr_workspace_bytes": (_size, [_i64, _i64, _i64, _size]),
    "scorch_hip_spmm_csr_f32": (ctypes.c_int, _SPMM),
    "scorch_hip_spmm_csr_f64": (ctypes.c_int, _SPMM),
    "scorch_hip_spmm_csr_i32": (ctypes.c_int, _SPMM),
    "scorch_hip_spmm_csr_i64": (ctypes.c_int, _SPMM),
    "scorch_hip_spmm_csr_f32_static": (ctypes.c_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "scorch_hip_csr_inspect": (ctypes.c_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "scorch_hip_spmm_csr_rows_f32": (ctypes.c_int, _SPMM_ROWS),
    "scorch_hip_spmm_csr_rows_f64": (ctypes.c_int, _SPMM_ROWS),
    "scorch_hip_spmm_csr_rows_i32": (ctypes.c_int, _SPMM_ROWS),
    "scorch_hip_spmm_csr_rows_i64": (ctypes.c_int, _SPMM_ROWS),
    "scorch_hip_spmm_csr_bounds_bytes": (_size, [_i64, _i64, _i64, _size]),
    "scorch_hip_spmm_csr_bounds": (ctypes.c_int, [_i64, _i64, _i64, _size, _ptr, _ptr, _size, _ptr]),
    "scorch_hip_spmm_csr_planned_f32": (ctypes.c_int, _SPMM_PLANNED),
    "scorch_hip_spmm_csr_planned_f64": (ctypes.c_int, _SPMM_PLANNED),
    "scorch_hip_spmm_csr_planned_i32": (ctypes.c_int, _SPMM_PLANNED),
    "scorch_hip_spmm_csr_planned_i64": (ctypes.c_int, _SPMM_PLANNED),
    "scorch_hip_dense_tiled_bytes": (_size, [_i64, _i64, _size]),
    "scorch_hip_dense_tiled_recommended": (ctypes.c_int, [_i64, _i64, _i64, _size]),
    "scorch_hip_dense_to_tiled_f32": (ctypes.c_int, [_i64, _i64, _ptr, _ptr, _size, _ptr]),
    "scorch_hip_spmm_csr_tiled_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _size, _ptr,
                                                     ctypes.c_int, _ptr, _ptr, _size, _ptr, _size, _i64, _ptr]),
    "scorch_hip_spmm_csr_f32_timed": (ctypes.c_int, _SPMM + [ctypes.POINTER(ctypes.c_float)]),
    "scorch_hip_spmm_csr_bias_act_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr,
                                                        _ptr, ctypes.c_int, _ptr, _ptr, _size, _ptr]),
    "scorch_hip_spgemm_csr_workspace_bytes": (_size, [_i64, _i64, _size]),
    "scorch_hip_spgemm_csr_symbolic": (ctypes.c_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                                      _size, _ptr]),
    "scorch_hip_spgemm_csr_numeric_f32": (ctypes.c_int, _SPGEMM),
    "scorch_hip_spgemm_csr_numeric_f64": (ctypes.c_int, _SPGEMM),
    "scorch_hip_spgemm_csr_numeric_i32": (ctypes.c_int, _SPGEMM),
    "scorch_hip_spgemm_csr_numeric_i64": (ctypes.c_int, _SPGEMM),
    "scorch_hip_sddmm_coo_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr,
                                                _ptr, _ptr]),
    "scorch_hip_sddmm_csr_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr,
                                                _ptr, _ptr, _ptr]),
    "scorch_hip_sddmm_csr_batched_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr,
                                                        _ptr, _ptr, _ptr]),
    "scorch_hip_softmax_csr_batched_f32": (ctypes.c_int, [_i64, _i64, _i64, _ptr, _ptr, ctypes.c_float, _ptr, _ptr,
                                                          _size, _ptr]),
    "scorch_hip_spmm_csr_rows_batched_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr,
                                                            _ptr, _ptr]),
    "scorch_hip_spmm_csr_batched_workspace_bytes": (_size, [_i64, _i64, _i64, _i64]),
    "scorch_hip_spmm_csr_batched_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr,
                                                       _ptr, _size, _ptr, _size, _ptr]),
    "scorch_hip_sddmm_csr_lists_bytes": (_size, [_i64]),
    "scorch_hip_sddmm_csr_lists": (ctypes.c_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _size, _ptr]),
    "scorch_hip_sddmm_csr_list_values_f32": (ctypes.c_int, [_i64, _ptr, _size, _ptr, _ptr, _ptr]),
    "scorch_hip_sddmm_csr_listed_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _ptr, _size, _ptr, _ptr, _ptr, _ptr,
                                                       _ptr, _ptr, _ptr]),
    "scorch_hip_spmv_csr_workspace_bytes": (_size, [_i64, _i64, _size]),
    "scorch_hip_spmv_csr_f32": (ctypes.c_int, _SPMV),
    "scorch_hip_spmv_csr_f64": (ctypes.c_int, _SPMV),
    "scorch_hip_spmv_csr_i32": (ctypes.c_int, _SPMV),
    "scorch_hip_spmv_csr_i64": (ctypes.c_int, _SPMV),
    "scorch_hip_softmax_csr_workspace_bytes": (_size, [_i64, _i64]),
    "scorch_hip_softmax_csr_f32": (ctypes.c_int, [_i64, _i64, _ptr, _ptr, ctypes.c_float, _ptr, _ptr, _size,
                                                  _ptr]),
    "scorch_hip_softmax_csr_known_rows_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _ptr, _ptr, ctypes.c_float, _ptr,
                                                             _ptr, ctypes.c_size_t, _ptr]),
    "scorch_hip_attn_blocksparse_bf16": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr,
                                                        _ptr, ctypes.c_float, _ptr, _ptr]),
    "scorch_hip_attn_blocksparse_masked_bf16": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64,
                                                               _ptr, _ptr, _ptr, _ptr, ctypes.c_float, _ptr,
                                                               _ptr]),
    "scorch_hip_attn_blocksparse_split_workspace_bytes": (_size, [_i64, _i64, _i64]),
    "scorch_hip_attn_blocksparse_split_bf16": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _i64, _ptr, ctypes.c_int, ctypes.c_int, _i64, _ptr, _i64,
                                                              _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, ctypes.c_float,
                                                              _ptr, _ptr, _size, _ptr]),
    "scorch_hip_attn_blocksparse_f32_workspace_bytes": (_size, [_i64, _i64, _i64]),
    "scorch_hip_attn_blocksparse_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _i64,
                                                       _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, ctypes.c_float, _ptr,
                                                       _ptr, _size, _ptr]),
    "scorch_hip_sddmm_csr_blocked_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr,
                                                        _ptr, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "scorch_hip_spmm_csr_blocked_workspace_bytes": (_size, [_i64, _i64, _i64]),
    "scorch_hip_spmm_csr_blocked_f32": (ctypes.c_int, [_i64, _i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _i64,
                                                       _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _size, _ptr]),
    "scorch_hip_csr_row_indices": (ctypes.c_int, [_i64, _i64, _ptr, _ptr, _ptr]),
    "scorch_hip_coo_row_ptr": (ctypes.c_int, [_i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "scorch_hip_values_differ_f32": (ctypes.c_int, [_i64, _ptr, ctypes.c_float, _ptr, _ptr]),
    "scorch_hip_csr_block_count": (ctypes.c_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "scorch_hip_csr_block_fill": (ctypes.c_int, [_i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr,
                                                 _ptr, _ptr]),
}

_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


class ScorchHipError(RuntimeError):
    """A libscorch_hip call returned a non-zero status."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libscorch_hip error {code}: {message}")
        self.code = code


def library_path() -> str:
    return _build.LIB_PATH


def lib() -> ctypes.CDLL:
    """The loaded library (built first if the file is missing)."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(_build.LIB_PATH):
                    _build.build_library()
                handle = ctypes.CDLL(_build.LIB_PATH)
                for name, (restype, argtypes) in SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype = restype
                    fn.argtypes = argtypes
                _lib = handle
    return _lib


def kernel_times(call):
    """Run ``call()`` (one library call, or several) and return the duration of each
    kernel it launched, in milliseconds, in launch order (scorch_hip_timing_begin /
    _end).  Synchronises."""
    L = lib()
    check(L.scorch_hip_timing_begin())
    try:
        call()
    finally:
        ms = (ctypes.c_float * 16)()
        n = ctypes.c_int(0)
        rc = L.scorch_hip_timing_end(ms, 16, ctypes.byref(n))
    check(rc)
    return [ms[i] for i in range(min(n.value, 16))]


def last_error() -> str:
    return lib().scorch_hip_last_error().decode("utf-8", "replace")


def check(code: int) -> None:
    if code != OK:
        raise ScorchHipError(code, last_error())
