"""The library's plan handle (scorch_hip_csr_plan_* in include/scorch_hip.h) for torch tensors.

    with CsrPlanHandle(row_ptr, col_idx, n_cols) as plan:
        for _ in range(layers):
            h = plan.spmm(vals, h)              # the library picks the kernel; nothing is re-inspected

This is the binding a host that keeps its own state per sparse operand would write: one object
per pattern, one call per product, the library deciding between its kernels.  The module-level
functions of scorch_ops_hip do the same bookkeeping in Python, tensor by tensor, because the
reference's module interface (src/scorch/prebuilt_kernels.py:198-224) has no object to hang a
plan on.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import native

PLAN_SPMM_F32, PLAN_SDDMM_F32, PLAN_SOFTMAX_F32, PLAN_SPMM_DENSE_F32 = 0, 1, 2, 3
ACT_NONE, ACT_RELU = 0, 1


def _stream(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


class DensePlanHandle:
    """Owns one scorch_hip_dense_plan: a dense fp32 operand (K, N) that many products use unchanged.
    Keeps the tensor alive; after writing new values into it call update() before the next product."""

    def __init__(self, B: torch.Tensor):
        if B.dim() != 2 or B.dtype != torch.float32 or not B.is_cuda or not B.is_contiguous():
            raise TypeError("DensePlanHandle: B must be a contiguous 2-D fp32 tensor on the GPU")
        self.B, self.device = B, B.device
        self.K, self.N = B.shape
        self._handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_dense_plan_create(self.K, self.N, B.data_ptr(), _stream(self.device),
                                                                   ctypes.byref(self._handle)))

    def update(self) -> None:
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_dense_plan_update(self._live(), _stream(self.device)))

    def close(self) -> None:
        handle, self._handle = self._handle, ctypes.c_void_p()
        if handle:
            native.check(native.lib().scorch_hip_dense_plan_destroy(handle))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _live(self):
        if not self._handle:
            raise RuntimeError("DensePlanHandle: the plan has been closed")
        return self._handle


class CsrPlanHandle:
    """Owns one scorch_hip_csr_plan.  Keeps the two index tensors alive (the library keeps their
    addresses, not copies); they must not be written to while the handle lives."""

    def __init__(self, row_ptr: torch.Tensor, col_idx: torch.Tensor, n_cols: int):
        for name, t in (("row_ptr", row_ptr), ("col_idx", col_idx)):
            if t.dtype != torch.int32 or not t.is_cuda or not t.is_contiguous():
                raise TypeError(f"CsrPlanHandle: {name} must be a contiguous int32 tensor on the GPU")
        if row_ptr.device != col_idx.device or row_ptr.numel() < 1:
            raise ValueError("CsrPlanHandle: row_ptr and col_idx must share a device; row_ptr has M + 1 entries")
        self.row_ptr, self.col_idx = row_ptr, col_idx
        self.device = row_ptr.device
        self.M, self.n_cols, self.nnz = row_ptr.numel() - 1, int(n_cols), col_idx.numel()
        self._handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_csr_plan_create(
                self.M, self.n_cols, self.nnz, row_ptr.data_ptr(), col_idx.data_ptr(), _stream(self.device),
                ctypes.byref(self._handle)))

    # -- lifetime ---------------------------------------------------------------
    def close(self) -> None:
        handle, self._handle = self._handle, ctypes.c_void_p()
        if handle:
            native.check(native.lib().scorch_hip_csr_plan_destroy(handle))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:       # interpreter shutdown: the process's memory goes anyway
            pass

    def _live(self):
        if not self._handle:
            raise RuntimeError("CsrPlanHandle: the plan has been closed")
        return self._handle

    # -- what the library found ---------------------------------------------------
    def info(self) -> dict:
        raw = (ctypes.c_int64 * 8)()
        native.check(native.lib().scorch_hip_csr_plan_info(self._live(), raw))
        return {"M": raw[0], "n_cols": raw[1], "nnz": raw[2], "longest_row": raw[3], "empty_rows": raw[4],
                "sorted_rows": bool(raw[5]), "device_bytes": raw[6]}

    def prepare(self, op: int, width: int = 0) -> None:
        """Allocate and compute now what products of kind `op` and this width need, so that
        they allocate nothing later (before a graph capture, for instance)."""
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_csr_plan_prepare(self._live(), op, width, _stream(self.device)))

    # -- products ---------------------------------------------------------------------
    def _f32(self, t: Optional[torch.Tensor], numel: int, what: str) -> Optional[int]:
        if t is None:
            return None
        if t.dtype != torch.float32 or t.device != self.device or not t.is_contiguous() or t.numel() != numel:
            raise ValueError(f"CsrPlanHandle: {what} must be a contiguous fp32 tensor of {numel} elements on "
                             f"{self.device}")
        return t.data_ptr()

    def spmm(self, vals: torch.Tensor, B: torch.Tensor, bias: Optional[torch.Tensor] = None,
             relu: bool = False) -> torch.Tensor:
        """act(A @ B + bias) for B of shape (n_cols, N)."""
        if B.dim() != 2 or B.shape[0] != self.n_cols:
            raise ValueError(f"CsrPlanHandle.spmm: B must be ({self.n_cols}, N)")
        if relu and bias is None:
            raise ValueError("CsrPlanHandle.spmm: the activation comes with a bias")
        N = B.shape[1]
        out = torch.empty((self.M, N), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_spmm_csr_plan_f32(
                self._live(), N, self._f32(vals, self.nnz, "vals"), self._f32(B, self.n_cols * N, "B"),
                self._f32(bias, N, "bias"), ACT_RELU if relu else ACT_NONE, out.data_ptr(), _stream(self.device)))
        return out

    def spmm_dense(self, vals: torch.Tensor, dense: DensePlanHandle, bias: Optional[torch.Tensor] = None,
                   relu: bool = False) -> torch.Tensor:
        """spmm() with the dense operand named by its plan (a weight matrix stored by column tiles
        where that pays)."""
        if relu and bias is None:
            raise ValueError("CsrPlanHandle.spmm_dense: the activation comes with a bias")
        out = torch.empty((self.M, dense.N), dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_spmm_csr_plan_dense_f32(
                self._live(), self._f32(vals, self.nnz, "vals"), dense._live(), self._f32(bias, dense.N, "bias"),
                ACT_RELU if relu else ACT_NONE, out.data_ptr(), _stream(self.device)))
        return out

    def sddmm(self, mask_vals: Optional[torch.Tensor], A: torch.Tensor, B: torch.Tensor,
              rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """mask_vals[p] * <A[i_p], B[j_p]> per stored entry (mask_vals None: a mask of ones);
        `rows`, an int32 tensor of nnz entries, receives every entry's row."""
        if A.dim() != 2 or B.dim() != 2 or A.shape[0] != self.M or B.shape[0] != self.n_cols \
                or A.shape[1] != B.shape[1]:
            raise ValueError(f"CsrPlanHandle.sddmm: A must be ({self.M}, K) and B ({self.n_cols}, K)")
        K = A.shape[1]
        if rows is not None and (rows.dtype != torch.int32 or rows.numel() != self.nnz or rows.device != self.device
                                 or not rows.is_contiguous()):
            raise ValueError("CsrPlanHandle.sddmm: rows must be a contiguous int32 tensor of nnz entries")
        out = torch.empty(self.nnz, dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_sddmm_csr_plan_f32(
                self._live(), K, self._f32(mask_vals, self.nnz, "mask_vals"), self._f32(A, self.M * K, "A"),
                self._f32(B, self.n_cols * K, "B"), out.data_ptr(), rows.data_ptr() if rows is not None else None,
                _stream(self.device)))
        return out

    def softmax(self, vals: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        out = torch.empty(self.nnz, dtype=torch.float32, device=self.device)
        with torch.cuda.device(self.device):
            native.check(native.lib().scorch_hip_softmax_csr_plan_f32(
                self._live(), self._f32(vals, self.nnz, "vals"), scale, out.data_ptr(), _stream(self.device)))
        return out
