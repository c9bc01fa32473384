"""Helpers shared by the dispatch modules (reference: src/scorch/utils.py)."""
from .format import parse_format  # noqa: F401  (same import path as the reference's utils.parse_format)


import torch


def check_csr_indices(row_ptr: torch.Tensor, col_idx: torch.Tensor, n_cols: int, what: str = "operand") -> None:
    """Raise ValueError unless (row_ptr, col_idx) is a well-formed CSR index for a
    matrix with ``n_cols`` columns: row_ptr starts at 0, never decreases and ends
    at len(col_idx); every column lies in [0, n_cols).

    Neither the reference's kernels nor the HIP kernels look at index contents: an
    out-of-range column is undefined behaviour on the host and a memory fault on a
    GPU.  This check runs with torch operations on whatever device holds the
    arrays (one pass over them plus a synchronisation) and names what is wrong;
    the device wrappers make the same checks with one kernel the first time they
    see an operand (scorch_ops_hip.csr_plan)."""
    if row_ptr.numel() == 0:
        raise ValueError(f"{what}: empty row pointer")
    problems = []
    if int(row_ptr[0]) != 0:
        problems.append(f"row_ptr[0] = {int(row_ptr[0])}, expected 0")
    if int(row_ptr[-1]) != col_idx.numel():
        problems.append(f"row_ptr[-1] = {int(row_ptr[-1])}, but there are {col_idx.numel()} column indices")
    if row_ptr.numel() > 1 and bool((row_ptr[1:] < row_ptr[:-1]).any()):
        problems.append("row_ptr decreases somewhere")
    if col_idx.numel():
        lo, hi = int(col_idx.min()), int(col_idx.max())
        if lo < 0 or hi >= n_cols:
            problems.append(f"column indices span [{lo}, {hi}], outside [0, {n_cols})")
    if problems:
        raise ValueError(f"{what}: malformed CSR index: " + "; ".join(problems))
