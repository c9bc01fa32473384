"""Device counterpart of the reference's pybind module ``scorch_ops``.

Same function names, same argument lists and the same shape of return value as
csrc/ops.cpp binds them -- ``fn(result_shape, A_shape, A_mode_indices,
A_values, B_shape, B_mode_indices, B_values[, ...])`` returning an object with
``.storage.value`` and ``.storage.index.mode_indices`` -- so the reference's
dispatch (src/scorch/prebuilt_kernels.py:198-224, src/scorch/ops.py:405-415,
src/scorch/trace.py:288-299) can call either module.  The tensors must live on
a HIP device; the work is done by libscorch_hip.so on the current stream of
the operands' device and the call returns without synchronising.

Every symbol of the reference's matmul registry has a counterpart here (CSR x
dense, CSR x vector, CSR x CSR and the two coordinate-form products) beside
the SDDMM and fused-epilogue symbols.

What the reference's stateless dispatch does not have: a sparse operand is
inspected the first time it is seen (index validation, longest row) and the
result, with the chunk boundaries of the merge-path kernels, is kept on the
operand's row-pointer tensor; a wide dense operand that comes back unchanged
is re-stored once by column tiles (see CsrPlan and _tiled_operand below).
"""
from __future__ import annotations

import math
import os
import weakref
from typing import Dict, Optional, Tuple

import torch

from . import native

# Every buffer this module allocates comes from these two names, so that a test can put a
# poisoning allocator in their place: no kernel may depend on what a fresh buffer holds.
_empty = torch.empty
_empty_like = torch.empty_like

HINT_MOSTLY_EMPTY_ROWS = 0x100      # SCORCH_HIP_HINT_MOSTLY_EMPTY_ROWS of include/scorch_hip.h
INSPECT_REPORT_INTS = 8             # SCORCH_HIP_INSPECT_REPORT_INTS
_SUFFIX = {torch.float32: "f32", torch.float64: "f64", torch.int32: "i32", torch.int64: "i64"}


class TensorIndex:
    __slots__ = ("mode_indices",)

    def __init__(self, mode_indices=None):
        self.mode_indices = mode_indices if mode_indices is not None else []


class TensorStorage:
    __slots__ = ("value", "index")

    def __init__(self, value=None, index=None):
        self.value = value
        self.index = index if index is not None else TensorIndex()


class Tensor:
    """Result carrier with the fields of the reference's csrc/header.h:4-16
    (``workspace``: scratch memory that must live as long as the result, see
    _workspace)."""
    __slots__ = ("storage", "workspace")

    def __init__(self, value=None, mode_indices=None):
        self.storage = TensorStorage(value, TensorIndex(mode_indices))
        self.workspace = None


# ---- helpers -----------------------------------------------------------------
_workspaces = {}


def _workspace(device: torch.device, stream: int, nbytes: int) -> torch.Tensor:
    """Scratch buffer for (device, stream), grown on demand.  Kernels on one
    stream run in order, so they can share it; host threads that launch on
    different streams get different buffers.  While the stream is being
    captured into a HIP graph the buffer comes fresh from the graph's own memory
    pool instead: a replay must not write into a block that eager calls on the
    same stream use, or that was replaced by a larger one and returned to the
    allocator since the capture."""
    if torch.cuda.is_current_stream_capturing():
        return _empty(max(nbytes, 256), dtype=torch.uint8, device=device)
    key = (device.index, stream)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = _empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def _device_of(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError("scorch_ops_hip: operands must be on a HIP device, got " + str(dev))
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError(f"scorch_ops_hip: operands on different devices ({dev} and {t.device})")
    return dev


def _index(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dtype != torch.int32:
        raise TypeError(f"scorch_ops_hip: {what} must be int32, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def _flat(t: torch.Tensor, dtype: torch.dtype, what: str) -> torch.Tensor:
    if t.dtype != dtype:
        raise TypeError(f"scorch_ops_hip: {what} must be {dtype}, got {t.dtype}")
    return t if t.is_contiguous() else t.contiguous()


def _csr_parts(mode_indices, what: str, n_cols: Optional[int] = None):
    if len(mode_indices) != 2 or len(mode_indices[1]) != 2:
        raise ValueError(f"scorch_ops_hip: {what} is not a CSR (\"d,s\") operand")
    pos, crd = _index(mode_indices[1][0], what + " pos"), _index(mode_indices[1][1], what + " crd")
    return pos, crd


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(dev: torch.device) -> int:
    """Handle of torch's current stream on `dev` (the raw getter costs a fraction of
    a microsecond; building a Stream object, several)."""
    if _raw_stream is not None:
        return _raw_stream(dev.index)
    return torch.cuda.current_stream(dev).cuda_stream


_code_loaded = set()     # devices on which scorch_hip_init has run


class _on_device:
    """``with _on_device(dev):`` makes `dev` the current device like
    ``torch.cuda.device`` does, but costs next to nothing when it already is."""
    __slots__ = ("index", "previous")

    def __init__(self, dev: torch.device):
        self.index = dev.index
        self.previous = -1

    def __enter__(self):
        current = torch.cuda.current_device()
        if current != self.index:
            self.previous = current
            torch.cuda.set_device(self.index)
        if self.index not in _code_loaded:
            # the library's device code, all of it, when a device is first used: otherwise the first
            # product of every kind pays for the part it is the first to need
            _code_loaded.add(self.index)
            native.check(native.lib().scorch_hip_init())
        return self

    def __exit__(self, *exc):
        if self.previous >= 0:
            torch.cuda.set_device(self.previous)
        return False


# ---- what is kept beside tensors between calls, and how a caller drops it ---------------------
# The reference's call is stateless (src/scorch/prebuilt_kernels.py:198-224); its only cache is keyed
# on the expression and the formats, never on values (src/scorch/ops.py:425-488).  This module keeps
# derived data as attributes of the tensors it was derived from:
#   from index tensors   the CsrPlan (validity, longest row, chunk boundaries, entry lists, block
#                        description), the row pointer of a coordinate mask, an attention mask's blocks
#   from value tensors   the column-tile copy of a wide dense operand, "this mask's values are all 1", a
#                        mask's values in the order of its SDDMM entry lists
# Each is stamped with the tensor's address, its version counter and its epoch (below), and rebuilt
# when the stamp no longer matches.  PyTorch bumps the version counter for every in-place operation
# of its own on the tensor or on a view of it.  It does not for writes through ``t.data``, a raw
# pointer, a numpy or DLPack alias, a kernel of another library, or the replay of a recorded graph:
# after such a write call forget(t), or mark the tensor volatile once.
_CACHE_ATTRIBUTES = ("_scorch_plan", "_scorch_tiled", "_scorch_seen", "_scorch_ones", "_scorch_listed", "_scorch_coo_pos",
                     "_scorch_block_mask", "_scorch_mask_checked", "_scorch_rows")


def _tensors_of(obj, seen=None):
    """The torch tensors reachable from `obj`: a tensor, an STensor (values and index arrays), a result
    carrier of this module, or lists / tuples / dicts of those."""
    if seen is None:
        seen = set()
    if obj is None or id(obj) in seen:
        return
    seen.add(id(obj))
    if isinstance(obj, torch.Tensor):
        yield obj
        origin = getattr(obj, "_scorch_origin", None)
        if origin is not None:
            yield from _tensors_of(origin, seen)
    elif isinstance(obj, (list, tuple)):
        for x in obj:
            yield from _tensors_of(x, seen)
    elif isinstance(obj, dict):
        for x in obj.values():
            yield from _tensors_of(x, seen)
    elif isinstance(obj, (Tensor, TensorStorage, TensorIndex)) or hasattr(obj, "storage"):
        storage = obj if isinstance(obj, TensorStorage) else getattr(obj, "storage", None)
        if isinstance(obj, TensorIndex):
            yield from _tensors_of(obj.mode_indices, seen)
        elif storage is not None:
            yield from _tensors_of(getattr(storage, "value", None), seen)
            yield from _tensors_of(getattr(getattr(storage, "index", None), "mode_indices", None), seen)


def _epoch(t: torch.Tensor) -> int:
    return getattr(t, "_scorch_epoch", 0)


def _stamp(t: torch.Tensor):
    """What must be unchanged for data derived from `t` to be served again."""
    return (t.data_ptr(), t._version, _epoch(t), t.numel())


def _same(ref, t: torch.Tensor) -> bool:
    """Whether the weak reference `ref` still names the tensor object `t`.  Derived data lives on
    one tensor of an operand (the row pointer) and names its partner (the column indices) by stamp;
    a stamp alone would also match another tensor that the allocator has since put at the freed
    partner's address."""
    return ref is not None and ref() is t


def forget(*objs) -> None:
    """Drop everything this module has derived from the given tensors (or from the tensors of the
    given STensors, results, lists): the next call inspects, plans and copies anew.  For writes that
    PyTorch's version counter does not see -- ``t.data``, raw pointers, numpy / DLPack aliases,
    kernels of other libraries, replays of recorded graphs."""
    for t in _tensors_of(objs):
        for name in _CACHE_ATTRIBUTES:
            if hasattr(t, name):
                try:
                    delattr(t, name)
                except AttributeError:
                    pass
        try:
            t._scorch_epoch = _epoch(t) + 1      # plans that live on a partner tensor name this one's epoch
        except (AttributeError, RuntimeError):
            pass


def mark_volatile(*objs, volatile: bool = True) -> None:
    """Tensors whose *values* change behind PyTorch's back (the static inputs and the results of a
    recorded graph, buffers another library writes): nothing derived from their values -- the
    column-tile copy, the all-ones verdict -- is kept or used from now on.  What is derived from an
    index tensor (a sparsity pattern) is not affected: use forget() when a pattern is rewritten."""
    for t in _tensors_of(objs):
        if volatile:
            for name in ("_scorch_tiled", "_scorch_seen", "_scorch_ones", "_scorch_listed"):
                if hasattr(t, name):
                    delattr(t, name)
        try:
            t._scorch_volatile = bool(volatile)
        except (AttributeError, RuntimeError):
            pass


def is_volatile(t: torch.Tensor) -> bool:
    return bool(getattr(t, "_scorch_volatile", False)) or \
        bool(getattr(getattr(t, "_scorch_origin", None), "_scorch_volatile", False))


# ---- what is computed once per operand ---------------------------------------------
def plans_enabled() -> bool:
    """Sparse operands are inspected and planned unless SCORCH_HIP_PLAN=0."""
    return os.environ.get("SCORCH_HIP_PLAN", "1") not in ("", "0")


ROWS_KERNEL_MAX_ROW = 256   # longest row for which the row-split kernel is chosen

# Which SpMM kernel serves a product.  "auto" (the default; SCORCH_HIP_SPMM_PATH
# overrides it at import) decides from the operand's plan; the other values pin one
# path whatever the operand looks like, for tests and measurements:
#   "rows"             the row-split kernel
#   "merge"            the merge-path kernels, with precomputed chunk boundaries
#   "merge_unplanned"  the merge-path kernels searching row_ptr in every wavefront
#   "tiled"            fp32 only: the dense operand re-stored by column tiles (built
#                      at once), merge-path split; other dtypes as "merge"
SPMM_PATHS = ("auto", "rows", "merge", "merge_unplanned", "tiled")
SPMM_PATH = os.environ.get("SCORCH_HIP_SPMM_PATH", "auto")


class CsrPlan:
    """Facts about one CSR index that do not change from call to call: it is well
    formed, its longest row, and (filled in on demand, per dense width) the
    chunk boundaries of the merge-path kernels.  Lives as an attribute of the
    row-pointer tensor, so it is dropped with the operand, and is rebuilt when
    either index tensor has been written to since."""
    __slots__ = ("key", "partner", "max_row", "empty_rows", "sorted_rows", "runs", "bounds", "sddmm_lists",
                 "sddmm_uses", "rows", "blocked", "blocked_uses")

    def __init__(self, key, max_row: int, empty_rows: int, sorted_rows: bool = False, runs: int = 0):
        self.key = key
        self.partner = None                                # weak reference to the column-index tensor (see _same)
        self.max_row = max_row
        self.empty_rows = empty_rows
        self.sorted_rows = sorted_rows                     # every row's column indices increase strictly
        self.runs = runs                                   # stretches of a row inside one aligned group of 64 columns
        self.bounds: Dict[Tuple[int, int], torch.Tensor] = {}
        self.sddmm_lists: Optional[torch.Tensor] = None   # the mask's entries listed per XCD (SDDMM)
        self.sddmm_uses = 0                                # SDDMM calls that could have used them
        self.rows: Optional[torch.Tensor] = None           # the row coordinate of every entry (SDDMM results)
        self.blocked = None                                # BlockedCsr, False (looked at: not blocky), None (not yet)
        self.blocked_uses = 0                              # products that could have gone to the block kernels


def csr_plan(pos: torch.Tensor, crd: torch.Tensor, n_rows: int, n_cols: int, what: str = "operand") -> Optional[CsrPlan]:
    """The plan of (pos, crd), built on first sight: one inspection kernel and
    one read of its four-integer report (a synchronisation).  Raises ValueError
    for a malformed index -- row pointers that do not start at 0, end at
    len(crd) or decrease, column indices outside [0, n_cols) -- before any
    kernel dereferences it.  None when planning is switched off or the stream
    is being captured (no synchronisation is possible there)."""
    key = (_stamp(pos), _stamp(crd), n_rows, n_cols)
    plan = getattr(pos, "_scorch_plan", None)
    if plan is not None and plan.key == key and _same(plan.partner, crd):
        return plan
    if not plans_enabled():
        return None
    if pos.numel() != n_rows + 1:
        raise ValueError(f"scorch_ops_hip: {what}: row pointer has {pos.numel()} entries, expected {n_rows + 1}")
    if torch.cuda.is_current_stream_capturing():
        return None
    dev = pos.device
    report = _empty(INSPECT_REPORT_INTS, dtype=torch.int32, device=dev)
    with _on_device(dev):
        native.check(native.lib().scorch_hip_csr_inspect(n_rows, n_cols, crd.numel(), pos.data_ptr(),
                                                         crd.data_ptr(), report.data_ptr(), _stream(dev)))
    bad_rows, bad_cols, max_row, empty_rows, descents, runs = report.tolist()[:6]
    if bad_rows or bad_cols:
        problems = []
        if bad_rows:
            problems.append(f"row_ptr must start at 0, never decrease and end at {crd.numel()}")
        if bad_cols:
            problems.append(f"a column index lies outside [0, {n_cols})")
        raise ValueError(f"scorch_ops_hip: {what}: malformed CSR index: " + "; ".join(problems))
    plan = CsrPlan(key, max_row, empty_rows, descents == 0, runs)
    plan.partner = weakref.ref(crd)
    try:
        pos._scorch_plan = plan
    except (AttributeError, RuntimeError):      # an object that takes no attributes: plan per call
        pass
    return plan


def _chunk_bounds(plan: CsrPlan, pos: torch.Tensor, M: int, nnz: int, N: int, elem: int, L, stream) -> torch.Tensor:
    """Chunk boundaries of the merge-path split for dense width N, computed once."""
    bounds = plan.bounds.get((N, elem))
    if bounds is None:
        bounds = _empty(L.scorch_hip_spmm_csr_bounds_bytes(M, nnz, N, elem), dtype=torch.uint8,
                             device=pos.device)
        native.check(L.scorch_hip_spmm_csr_bounds(M, nnz, N, elem, pos.data_ptr(), bounds.data_ptr(),
                                                  bounds.numel(), stream))
        plan.bounds[(N, elem)] = bounds
    return bounds


# A CSR operand whose entries cluster in 64 x 64 blocks (an attention mask) is multiplied on the
# fp32 matrix instruction, block by block, when its dense partner is 32, 64 or 128 wide.  "auto"
# (SCORCH_HIP_BLOCKED overrides it at import) decides when an operand comes back for its second
# product, from the share of the active blocks' positions that are stored; "off" keeps the
# general kernels, "always" takes the block kernels for every operand they can serve, however
# thinly filled, from its first product on.
BLOCKED_PATHS = ("auto", "off", "always")
BLOCKED_PATH = os.environ.get("SCORCH_HIP_BLOCKED", "auto")
# dense width -> share of the active blocks' positions that must be stored for the block kernels to
# be the faster ones (measured on uniformly filled 4,096 x 4,096 masks, 8 heads: the general
# kernels' time grows with the entries, the block kernels' with the blocks)
BLOCKED_MIN_FILL = {32: 0.17, 64: 0.15, 128: 0.12}
BLOCKED_WIDTHS = tuple(BLOCKED_MIN_FILL)
BLOCKED_STRETCH = 16         # blocks per work item at most
BLOCKED_STRETCHES = (16, 4, 1)   # the SDDMM's work items exist in these sizes: a small launch takes smaller ones
BLOCKED_MAX_BLOCKS = 1 << 24  # blocks of the whole matrix: beyond, the operand is a graph, not a mask
BLOCKED_MAX_NNZ = 1 << 27
BLOCKED_MAX_BLOCK_COLS = 1 << 17  # what scorch_hip_csr_block_count takes


class BlockedCsr:
    """A CSR pattern described by 64 x 64 blocks, for scorch_hip_{sddmm,spmm}_csr_blocked_f32:
    the active blocks in block row major order, per block and row a word of stored columns and
    the CSR position of the row's first entry in the block, and the two lists of work items."""
    __slots__ = ("n_active", "block_row_ptr", "block_col_idx", "block_words", "block_off", "block_cols", "block_nnz",
                 "sddmm_items", "spmm_items", "n_spmm_items", "spmm_split_rows", "n_spmm_split_rows", "n_spmm_slots",
                 "n_block_rows", "longest_block_row", "fill")


def _describe_blocks(pos: torch.Tensor, crd: torch.Tensor, M: int, n_cols: int, min_fill: float = 0.0):
    """(block_row_ptr on the host as a numpy array, the device arrays of scorch_hip_csr_block_fill) for
    the pattern (pos, crd): two kernel passes over the entries and, between them, one host read of
    the block rows' counts, which sizes the second pass's arrays.  None instead of the arrays when
    the active blocks hold less than `min_fill` of their positions (the second pass is then not run)."""
    L = native.lib()
    dev = pos.device
    nnz = int(crd.numel())
    nbr = M // 64
    block_row_ptr = _empty(nbr + 1, dtype=torch.int32, device=dev)
    with _on_device(dev):
        stream = _stream(dev)
        native.check(L.scorch_hip_csr_block_count(M, n_cols, nnz, pos.data_ptr(), crd.data_ptr(),
                                                  block_row_ptr.data_ptr(), stream))
        brp = block_row_ptr.cpu().numpy()                  # the one synchronisation
        n_active = int(brp[-1])
        if n_active == 0 or nnz < min_fill * n_active * 4096:
            return brp, None
        arrays = {
            "block_row_ptr": block_row_ptr,
            "block_col_idx": _empty(n_active, dtype=torch.int32, device=dev),
            "block_words": _empty(n_active * 64, dtype=torch.int64, device=dev),
            "block_off": _empty(n_active * 64, dtype=torch.int32, device=dev),
            "block_cols": _empty(n_active, dtype=torch.int64, device=dev),
            "block_nnz": _empty(n_active, dtype=torch.int32, device=dev),
        }
        native.check(L.scorch_hip_csr_block_fill(
            M, n_cols, nnz, pos.data_ptr(), crd.data_ptr(), block_row_ptr.data_ptr(), n_active,
            arrays["block_col_idx"].data_ptr(), arrays["block_words"].data_ptr(), arrays["block_off"].data_ptr(),
            arrays["block_cols"].data_ptr(), arrays["block_nnz"].data_ptr(), stream))
    return brp, arrays


def _stretches(lens, longest, split_slots: bool):
    """Work items (block row, begin, end, slot) over block rows of `lens` active blocks each, as an
    int32 array of shape (n, 4) sorted longest first (ties in row order): a block row with more
    than `longest` blocks goes out in ceil(n / longest) stretches of nearly equal length.  With
    `split_slots` a whole row's slot is -1 and the stretches of a shared-out row get consecutive
    slots, returned with the list of those rows (block row, first slot, stretches, 0) and the number
    of slots; otherwise the slot is 0."""
    import numpy as np
    lens = np.asarray(lens, dtype=np.int64)
    at = np.concatenate([[0], np.cumsum(lens)])[:-1]
    parts = np.maximum(-(-lens // max(int(longest), 1)), 1)
    row = np.repeat(np.arange(lens.size, dtype=np.int64), parts)
    part = np.arange(row.size, dtype=np.int64) - np.repeat(np.cumsum(parts) - parts, parts)
    lo = at[row] + lens[row] * part // parts[row]
    hi = at[row] + lens[row] * (part + 1) // parts[row]
    slot = np.zeros(row.size, dtype=np.int64)
    split_rows, n_slots = np.zeros((0, 4), dtype=np.int32), 0
    if split_slots:
        shared = parts > 1
        first_slot = np.cumsum(np.where(shared, parts, 0)) - np.where(shared, parts, 0)
        slot = np.where(shared[row], first_slot[row] + part, -1)
        n_slots = int(parts[shared].sum())
        rows = np.nonzero(shared)[0]
        split_rows = np.stack([rows, first_slot[rows], parts[rows], np.zeros_like(rows)], axis=1).astype(np.int32)
    order = np.argsort(-(hi - lo), kind="stable")          # longest first
    items = np.stack([row, lo, hi, slot], axis=1)[order].astype(np.int32)
    return items, split_rows, n_slots


def _blocked_csr(plan: "CsrPlan", pos: torch.Tensor, crd: torch.Tensor, M: int, n_cols: int,
                 min_fill: float) -> Optional[BlockedCsr]:
    """The block description of (pos, crd), or None when the pattern is not one the block kernels
    serve (dimensions not multiples of 64, rows not strictly increasing, blocks too thinly filled).
    The inspection has already counted the pattern's runs, which bound the blocks' fill from above:
    a graph is turned away here without a kernel.  Otherwise two kernel passes (_describe_blocks)
    and the work-item lists, computed on the host from the block rows' lengths."""
    block = 64
    nnz = int(crd.numel())
    if M % block or n_cols % block or nnz == 0 or nnz > BLOCKED_MAX_NNZ:
        return None
    nbr, nbc = M // block, n_cols // block
    if nbr * nbc > BLOCKED_MAX_BLOCKS or nbc > BLOCKED_MAX_BLOCK_COLS or nnz < min_fill * block * M:
        return None                                        # (every block row has a block, usually)
    if not plan.sorted_rows or nnz < min_fill * block * plan.runs:
        return None
    dev = pos.device
    brp, arrays = _describe_blocks(pos, crd, M, n_cols, min_fill)
    if arrays is None:
        return None
    import numpy as np
    lens = np.diff(brp).astype(np.int64)
    n_active = int(brp[-1])
    # Work items.  SDDMM: stretches of block rows, in several sizes (the entries do not depend on how
    # they are shared out, so a launch picks the size that fills the chip).  SpMM: a block row sums into
    # one tile of the result, so it stays whole unless the rows differ by more than a quarter of their
    # mean; then rows longer than the mean by more than a block (4 to BLOCKED_STRETCH blocks) go out in
    # stretches whose sums a second kernel adds up in order -- the same stretches whatever the number of
    # heads, so that a head's result does not depend on what it is batched with.
    mean = n_active / nbr
    longest = int(lens.max())
    spmm_longest = min(BLOCKED_STRETCH, max(4, -(-n_active // nbr) + 1)) if longest > 1.25 * mean else longest
    to_device = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).reshape(-1)
    bl = BlockedCsr()
    bl.n_active = n_active
    bl.block_row_ptr = arrays["block_row_ptr"]
    bl.block_col_idx = arrays["block_col_idx"]
    bl.block_words = arrays["block_words"]
    bl.block_off = arrays["block_off"]
    bl.block_cols = arrays["block_cols"]
    bl.block_nnz = arrays["block_nnz"]
    bl.sddmm_items = {}
    for stretch in BLOCKED_STRETCHES:
        items, _, _ = _stretches(lens, stretch, False)
        items = items[items[:, 2] > items[:, 1]]           # a block row without blocks has no entries to compute
        bl.sddmm_items[stretch] = (to_device(items), int(items.shape[0]))
    items, split_rows, n_slots = _stretches(lens, spmm_longest, True)
    bl.spmm_items = to_device(items)
    bl.n_spmm_items = int(items.shape[0])
    bl.spmm_split_rows = to_device(split_rows)
    bl.n_spmm_split_rows = int(split_rows.shape[0])
    bl.n_spmm_slots = n_slots
    bl.n_block_rows = nbr
    bl.longest_block_row = longest
    bl.fill = nnz / (n_active * block * block)
    return bl


def _blocked(plan: Optional[CsrPlan], pos, crd, M: int, n_cols: int, width: int) -> Optional[BlockedCsr]:
    """The operand's block description if products with it go to the block kernels.  Decided when
    the operand (the same index tensors, unchanged) comes back for a second product: describing
    a pattern costs a pass of torch operations over its entries, which an operand that is built
    anew for every call -- the probabilities of an attention head wrapped in a fresh STensor --
    would pay each time.  Never under a stream capture unless it was decided before."""
    if BLOCKED_PATH not in BLOCKED_PATHS:
        raise ValueError(f"scorch_ops_hip: BLOCKED_PATH is {BLOCKED_PATH!r}, expected one of {BLOCKED_PATHS}")
    if BLOCKED_PATH == "off" or plan is None or width not in BLOCKED_WIDTHS:
        return None
    if plan.blocked is None:
        plan.blocked_uses += 1
        if torch.cuda.is_current_stream_capturing() or (plan.blocked_uses < 2 and BLOCKED_PATH != "always"):
            return None
        least = 0.0 if BLOCKED_PATH == "always" else min(BLOCKED_MIN_FILL.values())
        plan.blocked = _blocked_csr(plan, pos, crd, M, n_cols, least) or False
    bl = plan.blocked or None
    if bl is not None and BLOCKED_PATH == "auto" and bl.fill < BLOCKED_MIN_FILL[width]:
        return None
    return bl


def _blocked_sddmm(L, bl: BlockedCsr, heads: int, M: int, n_cols: int, K: int, nnz: int, mask_vals,
                   a: torch.Tensor, b: torch.Tensor, out: torch.Tensor, rows_ptr, stream: int) -> int:
    """Launch the block SDDMM for `heads` pairs of dense operands over one pattern: with the
    largest work items that still give every workgroup slot of the chip one (1,024: 256 CUs x 4),
    else the smallest."""
    for stretch in BLOCKED_STRETCHES:
        items, n_items = bl.sddmm_items[stretch]
        if n_items * heads >= 1024:
            break
    return L.scorch_hip_sddmm_csr_blocked_f32(
        heads, M, n_cols, K, nnz, bl.n_active, bl.block_col_idx.data_ptr(), bl.block_words.data_ptr(),
        bl.block_off.data_ptr(), n_items, items.data_ptr(),
        _mask_values_pointer(mask_vals), a.data_ptr(), b.data_ptr(), out.data_ptr(), rows_ptr, stream)


def _mask_values_pointer(values: Optional[torch.Tensor]):
    """What an SDDMM kernel is handed for its mask's values: nothing when they are known to be all 1
    (the kernel then reads nothing for them), else the array."""
    return None if values is None or _known_all_ones(values) else values.data_ptr()


def _listed_mask_values(values: torch.Tensor, lists: torch.Tensor, L, stream):
    """What the listed SDDMM kernel is handed for its mask's values: (mask_vals, listed_vals)
    pointers.  Nothing at all when the values are known to be all 1; the values in the order of the
    lists (read with the entries, coalesced) once the same unchanged tensor has come back and has
    been found not to be all ones -- one gather, kept with the tensor; else the array itself (one
    scattered load per entry).  Never a copy while a stream is capturing or for a volatile tensor:
    a recording holds pointers, and the values may be rewritten before a replay."""
    if _known_all_ones(values):
        return None, None
    if torch.cuda.is_current_stream_capturing() or is_volatile(values):
        return values.data_ptr(), None
    key = _stamp(values)
    cached = getattr(values, "_scorch_listed", None)
    if cached is not None and cached[0] == key and cached[1] is lists:
        return values.data_ptr(), cached[2].data_ptr()
    seen = getattr(values, "_scorch_ones", None)
    if seen is None or seen[0] != key or seen[1] is not False:
        return values.data_ptr(), None          # not yet seen twice unchanged
    listed = _empty_like(values)
    native.check(L.scorch_hip_sddmm_csr_list_values_f32(values.numel(), lists.data_ptr(), lists.numel(),
                                                        values.data_ptr(), listed.data_ptr(), stream))
    try:
        values._scorch_listed = (key, lists, listed)
    except (AttributeError, RuntimeError):
        return values.data_ptr(), None
    return values.data_ptr(), listed.data_ptr()


def _known_all_ones(values: torch.Tensor) -> bool:
    """Whether a mask's values are known to be all 1 (an attention mask; the block SDDMM then
    reads nothing for them).  Looked at when the same tensor comes back unchanged -- one
    reduction and one read of its result -- and remembered with the tensor."""
    if torch.cuda.is_current_stream_capturing() or is_volatile(values):
        # a recording holds pointers, not verdicts: the values may be rewritten before a replay
        return False
    key = _stamp(values)
    seen = getattr(values, "_scorch_ones", None)
    if seen is not None and seen[0] == key:
        if seen[1] is None:
            differ = _empty(1, dtype=torch.int32, device=values.device)
            with _on_device(values.device):
                native.check(native.lib().scorch_hip_values_differ_f32(values.numel(), values.data_ptr(), 1.0,
                                                                       differ.data_ptr(), _stream(values.device)))
            seen = (key, values.dtype == torch.float32 and not differ.item())
            values._scorch_ones = seen
        return bool(seen[1])
    try:
        values._scorch_ones = (key, None)
    except (AttributeError, RuntimeError):
        pass
    return False


def _blocked_spmm(L, bl: BlockedCsr, heads: int, M: int, K: int, N: int, nnz: int, vals: torch.Tensor,
                  b: torch.Tensor, out: torch.Tensor, stream: int) -> int:
    """Launch the block SpMM for `heads` value arrays over one pattern."""
    ws = None
    if bl.n_spmm_slots:
        ws = _workspace(out.device, stream, L.scorch_hip_spmm_csr_blocked_workspace_bytes(heads, bl.n_spmm_slots, N))
        if torch.cuda.is_current_stream_capturing():
            out._scorch_workspace = ws      # a buffer handed out during a capture lives as long as the result
    return L.scorch_hip_spmm_csr_blocked_f32(
        heads, M, K, N, nnz, bl.n_active, bl.block_col_idx.data_ptr(), bl.block_words.data_ptr(),
        bl.block_off.data_ptr(), bl.block_cols.data_ptr(), bl.n_spmm_items, bl.spmm_items.data_ptr(),
        bl.n_spmm_split_rows,
        bl.spmm_split_rows.data_ptr() if bl.n_spmm_split_rows else None, bl.n_spmm_slots, vals.data_ptr(),
        b.data_ptr(), out.data_ptr(), ws.data_ptr() if ws is not None else None,
        ws.numel() if ws is not None else 0, stream)


def tiled_operands_enabled() -> bool:
    """A wide dense operand that is multiplied again unchanged is re-stored by
    column tiles unless SCORCH_HIP_TILED=0."""
    return os.environ.get("SCORCH_HIP_TILED", "1") not in ("", "0")


def _dense_owner(values: torch.Tensor) -> torch.Tensor:
    """The tensor object that carries a dense operand's cached layouts: the user's
    own tensor when `values` is the flat view STensor.from_torch made of it."""
    return getattr(values, "_scorch_origin", values)


def prepare_dense_operand(values: torch.Tensor, K: int, N: int) -> Optional[torch.Tensor]:
    """Store a dense fp32 operand (K x N, row-major, on a HIP device) by column
    tiles now, for the products that follow (what a second product with the same
    unchanged tensor would trigger by itself).  Returns the tiled copy, which
    stays attached to the tensor until the tensor is written to or dropped; None
    if the layout does not apply (other dtypes)."""
    if values.dtype != torch.float32:
        return None
    owner = _dense_owner(values)
    dev = values.device
    L = native.lib()
    flat = values if values.is_contiguous() else values.contiguous()
    bt = _empty(L.scorch_hip_dense_tiled_bytes(K, N, 4) // 4, dtype=torch.float32, device=dev)
    with _on_device(dev):
        native.check(L.scorch_hip_dense_to_tiled_f32(K, N, flat.data_ptr(), bt.data_ptr(), bt.numel() * 4,
                                                     _stream(dev)))
    owner._scorch_tiled = (owner._version, values.data_ptr(), K, N, bt, _epoch(owner))
    return bt


def _tiled_operand(values: torch.Tensor, K: int, N: int, nnz: int, L) -> Optional[torch.Tensor]:
    """The column-tile copy of a dense operand if it has one that is still valid,
    or if this is the second product in a row with the same unchanged tensor
    (then it is built now); else None.  Only for shapes where the layout pays."""
    if N < 512 or values.dtype != torch.float32:      # (rows of 2 KiB and more: the library's own first test)
        return None
    if not tiled_operands_enabled() or not L.scorch_hip_dense_tiled_recommended(K, N, nnz, 4):
        return None
    if torch.cuda.is_current_stream_capturing():
        # a copy of the operand's values must not be recorded into a graph: a replay after the
        # operand has been rewritten in place would read the old values, with nothing to notice it
        return None
    owner = _dense_owner(values)
    if is_volatile(owner) or is_volatile(values):
        return None
    stamp = (owner._version, values.data_ptr(), K, N)
    cached = getattr(owner, "_scorch_tiled", None)
    if cached is not None and cached[:4] == stamp and cached[5] == _epoch(owner):
        return cached[4]
    stamp = stamp + (_epoch(owner),)
    if getattr(owner, "_scorch_seen", None) == stamp:
        return prepare_dense_operand(values, K, N)
    try:
        owner._scorch_seen = stamp
    except (AttributeError, RuntimeError):
        pass
    return None


# ---- SpMM ----------------------------------------------------------------------
def _spmm(dtype, result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values,
          bias=None, act=0):
    M, K = int(A_shape[0]), int(A_shape[1])
    N = int(B_shape[1])
    if int(B_shape[0]) != K or len(result_shape) != 2 or int(result_shape[0]) != M or int(result_shape[1]) != N:
        raise ValueError(f"scorch_ops_hip: shape mismatch A{tuple(A_shape)} B{tuple(B_shape)} "
                         f"result{tuple(result_shape)}")
    pos, crd = _csr_parts(A_mode_indices, "A")
    a_val = _flat(A_values, dtype, "A values")
    b_val = _flat(B_values, dtype, "B values")
    if pos.numel() != M + 1 or b_val.numel() != K * N or crd.numel() != a_val.numel():
        raise ValueError("scorch_ops_hip: array lengths do not match the shapes")
    dev = _device_of(pos, crd, a_val, b_val)
    nnz = a_val.numel()
    bias_ptr = None
    if bias is not None:
        if dtype != torch.float32:
            raise TypeError("scorch_ops_hip: the fused bias / activation kernels are fp32")
        bias = _flat(bias, dtype, "bias")
        if bias.numel() != N or bias.device != dev:
            raise ValueError("scorch_ops_hip: bias must have N elements on the operands' device")
        bias_ptr = bias.data_ptr()
    if SPMM_PATH not in SPMM_PATHS:
        raise ValueError(f"scorch_ops_hip: SPMM_PATH is {SPMM_PATH!r}, expected one of {SPMM_PATHS}")
    plan = csr_plan(pos, crd, M, K, "A")
    out = _empty(M * N, dtype=dtype, device=dev)
    L = native.lib()
    suffix = _SUFFIX[dtype]
    elem = a_val.element_size()
    path = SPMM_PATH if M > 0 and N > 0 else "merge_unplanned"
    with _on_device(dev):
        stream = _stream(dev)
        # a wide dense operand that keeps coming back is served from its column-tile copy
        tiled = None
        if path == "auto":
            tiled = _tiled_operand(B_values, K, N, nnz, L)
        elif path == "tiled" and dtype == torch.float32:
            tiled = prepare_dense_operand(B_values, K, N)
        # most rows empty and a result large enough for two more launches not to show: one streaming
        # fill of the result, then only the rows that have entries (merge-path kernel)
        fill_first = plan is not None and bias is None and 2 * plan.empty_rows >= M and M * N * elem >= (32 << 20)
        if path == "auto" and tiled is None and dtype == torch.float32 and bias is None and act == 0:
            bl = _blocked(plan, pos, crd, M, K, N)
            if bl is not None:
                native.check(_blocked_spmm(L, bl, 1, M, K, N, nnz, a_val, b_val, out, stream))
                return Tensor(out, [[], []])
        if tiled is None and (path == "rows" or (path == "auto" and plan is not None and not fill_first
                                                 and plan.max_row <= ROWS_KERNEL_MAX_ROW)):
            # every row is short: one launch of the row-split kernel, no workspace
            rc = getattr(L, "scorch_hip_spmm_csr_rows_" + suffix)(
                M, K, N, nnz, pos.data_ptr(), crd.data_ptr(), a_val.data_ptr(), b_val.data_ptr(), bias_ptr, act,
                out.data_ptr(), stream)
            native.check(rc)
            return Tensor(out, [[], []])
        ws = _workspace(dev, stream, L.scorch_hip_spmm_csr_workspace_bytes(M, nnz, N, elem))
        bounds = _chunk_bounds(plan, pos, M, nnz, N, elem, L, stream) \
            if plan is not None and path != "merge_unplanned" else None
        bounds_ptr, bounds_bytes = (bounds.data_ptr(), bounds.numel()) if bounds is not None else (None, 0)
        if tiled is not None:
            rc = L.scorch_hip_spmm_csr_tiled_f32(M, K, N, nnz, pos.data_ptr(), crd.data_ptr(), a_val.data_ptr(),
                                                 tiled.data_ptr(), tiled.numel() * 4, bias_ptr, act, out.data_ptr(),
                                                 bounds_ptr, bounds_bytes, ws.data_ptr(), ws.numel(),
                                                 plan.max_row if plan is not None else 0, stream)
        else:
            hint = HINT_MOSTLY_EMPTY_ROWS if fill_first else 0
            rc = getattr(L, "scorch_hip_spmm_csr_planned_" + suffix)(
                M, K, N, nnz, pos.data_ptr(), crd.data_ptr(), a_val.data_ptr(), b_val.data_ptr(), bias_ptr,
                act | hint, out.data_ptr(), bounds_ptr, bounds_bytes, ws.data_ptr(), ws.numel(), stream)
    native.check(rc)
    result = Tensor(out, [[], []])
    result.workspace = ws      # a buffer handed out during a graph capture lives as long as the result
    return result


def _make_spmm(dtype):
    def kernel(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values,
               tile_size: int = 0):
        return _spmm(dtype, result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices,
                     B_values)
    return kernel


# fp32: the symbol the registry tries first, its typed fallback and the legacy alias
# (src/scorch/prebuilt_kernels.py:45); one kernel serves all three.
spmm_csr_float_v2 = _make_spmm(torch.float32)
prebuilt_spmm_csr_f32 = _make_spmm(torch.float32)
spmm_csr_float = _make_spmm(torch.float32)
prebuilt_spmm_csr_f64 = _make_spmm(torch.float64)
spmm_csr_double = _make_spmm(torch.float64)
prebuilt_spmm_csr_i32 = _make_spmm(torch.int32)
prebuilt_spmm_csr_i64 = _make_spmm(torch.int64)

# The reference also binds its CPU tiling experiments of the same fp32 product under
# names of their own (csrc/ops.cpp:121-160; called from its benchmark scripts and
# tests/test_scorch/test_perf_large.py).  A tiling for caches and SIMD units of a host
# has no meaning here: every name runs the one device kernel, tile arguments ignored.
SPMM_CSR_FLOAT_VARIANTS = ("optimized", "turbo", "ultra", "apex", "untiled", "direct", "neon", "row_panel",
                           "k_parallel", "sorted_rows", "neon2", "neon4", "tiled_neon")
for _variant in SPMM_CSR_FLOAT_VARIANTS:
    globals()["spmm_csr_float_" + _variant] = _make_spmm(torch.float32)
del _variant


def spmm_csr_float_tiled_i_k(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices,
                             B_values, i_tile_size: int = 0, k_tile_size: int = 0):
    return _spmm(torch.float32, result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices,
                 B_values)


def spmm_csr_bias_float(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices,
                        B_values, bias):
    """C = A @ B + bias (reference: csrc/ops.cpp:179-188)."""
    return _spmm(torch.float32, result_shape, A_shape, A_mode_indices, A_values, B_shape,
                 B_mode_indices, B_values, bias=bias, act=0)


def spmm_csr_bias_relu_float(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices,
                             B_values, bias):
    """C = relu(A @ B + bias) (reference: csrc/ops.cpp:168-177)."""
    return _spmm(torch.float32, result_shape, A_shape, A_mode_indices, A_values, B_shape,
                 B_mode_indices, B_values, bias=bias, act=1)


# ---- SpGEMM --------------------------------------------------------------------
def _make_spgemm(dtype):
    def kernel(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values):
        """C = A @ B, all CSR (reference: csrc/kernels.h:52-202).  Two kernels
        passes with one host read of the result size in between."""
        M, K, N = int(A_shape[0]), int(A_shape[1]), int(B_shape[1])
        if int(B_shape[0]) != K:
            raise ValueError(f"scorch_ops_hip: shape mismatch A{tuple(A_shape)} B{tuple(B_shape)}")
        a_pos, a_crd = _csr_parts(A_mode_indices, "A")
        b_pos, b_crd = _csr_parts(B_mode_indices, "B")
        a_val = _flat(A_values, dtype, "A values")
        b_val = _flat(B_values, dtype, "B values")
        if a_pos.numel() != M + 1 or b_pos.numel() != K + 1 or a_crd.numel() != a_val.numel() \
                or b_crd.numel() != b_val.numel():
            raise ValueError("scorch_ops_hip: array lengths do not match the shapes")
        dev = _device_of(a_pos, a_crd, a_val, b_pos, b_crd, b_val)
        csr_plan(a_pos, a_crd, M, K, "A")      # validates the indices (once per operand)
        csr_plan(b_pos, b_crd, K, N, "B")
        L = native.lib()
        with _on_device(dev):
            stream = _stream(dev)
            need = L.scorch_hip_spgemm_csr_workspace_bytes(M, N, a_val.element_size())
            ws = _workspace(dev, stream, need)
            c_pos = _empty(M + 1, dtype=torch.int32, device=dev)
            native.check(L.scorch_hip_spgemm_csr_symbolic(M, K, N, a_pos.data_ptr(), a_crd.data_ptr(),
                                                          b_pos.data_ptr(), b_crd.data_ptr(),
                                                          c_pos.data_ptr(), ws.data_ptr(), ws.numel(),
                                                          stream))
            nnz = int(c_pos[-1].item())
            if nnz < 0:
                raise native.ScorchHipError(native.EUNSUPPORTED,
                                            "SpGEMM: the result has 2^31 entries or more, beyond its int32 row pointer")
            c_crd = _empty(nnz, dtype=torch.int32, device=dev)
            c_val = _empty(nnz, dtype=dtype, device=dev)
            fn = getattr(L, "scorch_hip_spgemm_csr_numeric_" + _SUFFIX[dtype])
            native.check(fn(M, K, N, a_pos.data_ptr(), a_crd.data_ptr(), a_val.data_ptr(),
                            b_pos.data_ptr(), b_crd.data_ptr(), b_val.data_ptr(), c_pos.data_ptr(),
                            c_crd.data_ptr(), c_val.data_ptr(), ws.data_ptr(), ws.numel(), stream))
        return Tensor(c_val, [[], [c_pos, c_crd]])
    return kernel


_spgemm_f32_atomic = _make_spgemm(torch.float32)

# fp32 CSR x CSR sums are accumulated with floating-point atomics, so their last bits depend
# on the order in which the hardware happens to serve them.  With SPGEMM_REPRODUCIBLE (default:
# SCORCH_HIP_SPGEMM_REPRODUCIBLE) the fp32 product is computed in 64-bit fixed point instead,
# where addition is associative: the same bits on every run, whatever the order.
SPGEMM_REPRODUCIBLE = os.environ.get("SCORCH_HIP_SPGEMM_REPRODUCIBLE", "0") not in ("", "0")


def spmspm_csr_f32_reproducible(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values):
    """C = A @ B, all CSR, fp32 values, with sums that do not depend on the order of the
    additions: both operands are rounded to fixed point (A to multiples of 2^-sa, B of 2^-sb),
    multiplied with the exact int64 kernel, and the sums scaled back.  sa and sb are the largest
    shifts for which no row's sum can overflow: with P the largest number of products in a row,
    each operand keeps (62 - ceil(log2 P)) / 2 bits below its largest magnitude -- 23 bits, fp32's
    own, for P up to 65,536.  An entry's error is at most P * 2^-(bits) * max|A| * max|B|; small
    entries of operands with a wide range of magnitudes lose relative precision.  Same structure
    as the default mode (reference: csrc/kernels.h:52-202)."""
    M, K, N = int(A_shape[0]), int(A_shape[1]), int(B_shape[1])
    a_pos, a_crd = _csr_parts(A_mode_indices, "A")
    b_pos, b_crd = _csr_parts(B_mode_indices, "B")
    a_val, b_val = _flat(A_values, torch.float32, "A values"), _flat(B_values, torch.float32, "B values")
    if a_pos.numel() != M + 1 or b_pos.numel() != K + 1 or a_crd.numel() != a_val.numel() \
            or b_crd.numel() != b_val.numel():
        raise ValueError("scorch_ops_hip: array lengths do not match the shapes")
    dev = _device_of(a_pos, a_crd, a_val, b_pos, b_crd, b_val)
    csr_plan(a_pos, a_crd, M, K, "A")
    if a_val.numel() == 0 or b_val.numel() == 0:
        return _spgemm_f32_atomic(result_shape, A_shape, A_mode_indices, a_val, B_shape, B_mode_indices, b_val)
    if not (bool(torch.isfinite(a_val).all()) and bool(torch.isfinite(b_val).all())):
        raise ValueError("scorch_ops_hip: the reproducible SpGEMM needs finite values")
    # most products in one row of C: sum over the row's entries of the lengths of the B rows they select
    b_len = (b_pos[1:] - b_pos[:-1]).to(torch.int64)
    per_entry = b_len[a_crd.long()]
    rows = csr_row_indices(a_pos, int(a_crd.numel())).long()
    most = int(torch.zeros(M, dtype=torch.int64, device=dev).index_add_(0, rows, per_entry).max())
    bits = (62 - max(most, 1).bit_length()) // 2
    a_max, b_max = float(a_val.abs().max()), float(b_val.abs().max())

    def fixed(values, largest):
        if largest == 0.0:
            return torch.zeros(values.shape, dtype=torch.int64, device=dev), 0
        shift = bits - (math.frexp(largest)[1])        # |values| * 2^shift < 2^bits
        return torch.round(torch.ldexp(values.double(), torch.tensor(shift, device=dev))).to(torch.int64), shift

    a_fix, sa = fixed(a_val, a_max)
    b_fix, sb = fixed(b_val, b_max)
    out = prebuilt_spmspm_csr_i64(result_shape, A_shape, A_mode_indices, a_fix, B_shape, B_mode_indices, b_fix)
    c_fix = out.storage.value
    c_val = torch.ldexp(c_fix.double(), torch.tensor(-(sa + sb), device=dev)).to(torch.float32)
    return Tensor(c_val, out.storage.index.mode_indices)


def _spgemm_f32(*args):
    return spmspm_csr_f32_reproducible(*args) if SPGEMM_REPRODUCIBLE else _spgemm_f32_atomic(*args)


def prebuilt_spmspm_csr_f32(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values):
    """C = A @ B, all CSR, fp32 (reference: csrc/kernels.h:52-202).  Sums by floating-point
    atomics unless SPGEMM_REPRODUCIBLE is set (see spmspm_csr_f32_reproducible)."""
    return _spgemm_f32(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values)


def spmspm_csr_float(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values):
    return _spgemm_f32(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values)


prebuilt_spmspm_csr_f64 = _make_spgemm(torch.float64)
prebuilt_spmspm_csr_i32 = _make_spgemm(torch.int32)
prebuilt_spmspm_csr_i64 = _make_spgemm(torch.int64)


# ---- SpMV ----------------------------------------------------------------------
def _make_spmv(dtype):
    def kernel(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values):
        M, K = int(A_shape[0]), int(A_shape[1])
        pos, crd = _csr_parts(A_mode_indices, "A")
        a_val = _flat(A_values, dtype, "A values")
        x = _flat(B_values, dtype, "x values")
        if pos.numel() != M + 1 or x.numel() != K or crd.numel() != a_val.numel():
            raise ValueError("scorch_ops_hip: array lengths do not match the shapes")
        dev = _device_of(pos, crd, a_val, x)
        csr_plan(pos, crd, M, K, "A")
        y = _empty(M, dtype=dtype, device=dev)
        L = native.lib()
        with _on_device(dev):
            stream = _stream(dev)
            ws = _workspace(dev, stream, L.scorch_hip_spmv_csr_workspace_bytes(M, a_val.numel(),
                                                                              a_val.element_size()))
            fn = getattr(L, "scorch_hip_spmv_csr_" + _SUFFIX[dtype])
            rc = fn(M, K, a_val.numel(), pos.data_ptr(), crd.data_ptr(), a_val.data_ptr(), x.data_ptr(),
                    y.data_ptr(), ws.data_ptr(), ws.numel(), stream)
        native.check(rc)
        return Tensor(y, [[]])
    return kernel


prebuilt_spmv_csr_f32 = _make_spmv(torch.float32)
prebuilt_spmv_csr_f64 = _make_spmv(torch.float64)
prebuilt_spmv_csr_i32 = _make_spmv(torch.int32)
prebuilt_spmv_csr_i64 = _make_spmv(torch.int64)


SDDMM_PATHS = ("auto", "plain", "listed")
# "auto": a CSR mask seen for the second time, with a dense right operand between 8 and 20 MB
# (beyond one L2, within the eight together), is served from per-XCD entry lists; "plain" /
# "listed" pin one path (SCORCH_HIP_SDDMM_PATH sets the default).
SDDMM_PATH = os.environ.get("SCORCH_HIP_SDDMM_PATH", "auto")


def _sddmm_lists(plan: Optional[CsrPlan], pos, crd, M: int, n_cols: int, K: int, L, stream) -> Optional[torch.Tensor]:
    """The mask's per-XCD entry lists if this product should use them (built on the
    second such product with the mask), else None."""
    if SDDMM_PATH not in SDDMM_PATHS:
        raise ValueError(f"scorch_ops_hip: SDDMM_PATH is {SDDMM_PATH!r}, expected one of {SDDMM_PATHS}")
    if SDDMM_PATH == "plain" or plan is None or K > 256 or K == 0 or crd.numel() == 0:
        return None
    if SDDMM_PATH == "auto":
        b_bytes = n_cols * K * 4
        if not (8 << 20) <= b_bytes <= (20 << 20) or crd.numel() < 4 * n_cols:
            return None
        plan.sddmm_uses += 1
        if plan.sddmm_lists is None and (plan.sddmm_uses < 2 or torch.cuda.is_current_stream_capturing()):
            return None
    if plan.sddmm_lists is None:
        lists = _empty(L.scorch_hip_sddmm_csr_lists_bytes(crd.numel()), dtype=torch.uint8, device=pos.device)
        native.check(L.scorch_hip_sddmm_csr_lists(M, n_cols, crd.numel(), pos.data_ptr(), crd.data_ptr(),
                                                  lists.data_ptr(), lists.numel(), stream))
        plan.sddmm_lists = lists
    return plan.sddmm_lists


# ---- SDDMM ---------------------------------------------------------------------
def _sddmm_dense_args(S_shape, A_shape, A_values, B_shape, B_values):
    M, n_cols = int(S_shape[0]), int(S_shape[1])
    K = int(A_shape[1])
    if int(A_shape[0]) != M or int(B_shape[0]) != n_cols or int(B_shape[1]) != K:
        raise ValueError(f"scorch_ops_hip: shape mismatch S{tuple(S_shape)} A{tuple(A_shape)} "
                         f"B{tuple(B_shape)} (B is indexed [j, k])")
    a = _flat(A_values, torch.float32, "A values")
    b = _flat(B_values, torch.float32, "B values")
    if a.numel() != M * K or b.numel() != n_cols * K:
        raise ValueError("scorch_ops_hip: dense operand length does not match its shape")
    return M, n_cols, K, a, b


def _coo_mask_row_ptr(row: torch.Tensor, col: torch.Tensor, M: int, n_cols: int, K: int) -> Optional[torch.Tensor]:
    """The row pointer of a coordinate mask that may be one for the block kernels (dimensions
    multiples of 64, a dense width they serve, eight entries per row or more), once the same
    coordinate tensors have come back unchanged; None otherwise, and for coordinates that are
    not in row order.  Kept with the row tensor (one kernel and one host read, once)."""
    if BLOCKED_PATH == "off" or not plans_enabled() or K not in BLOCKED_WIDTHS or M % 64 or n_cols % 64 \
            or row.numel() < 8 * M or M == 0:
        return None
    key = (_stamp(row), _stamp(col), M)
    seen = getattr(row, "_scorch_coo_pos", None)
    if seen is not None and seen[0] == key and _same(seen[2], col):
        if seen[1] is None and not torch.cuda.is_current_stream_capturing():
            pos = coo_row_ptr(row, M)
            seen = (key, pos if pos is not None else False, seen[2])
            row._scorch_coo_pos = seen
            if pos is not None:
                plan = csr_plan(pos, col, M, n_cols, "S")
                if plan is not None:
                    plan.blocked_uses = 1           # this is the mask's second product already
        return seen[1] if isinstance(seen[1], torch.Tensor) else None
    try:
        row._scorch_coo_pos = (key, None, weakref.ref(col))
    except (AttributeError, RuntimeError):
        pass
    return None


def sddmm_coo_float_prebuilt(result_shape, S_shape, S_mode_indices, S_values, A_shape, A_mode_indices,
                             A_values, B_shape, B_mode_indices, B_values):
    """D = S * (A @ B^T) at S's entries, S in coordinate format
    (reference: csrc/kernels.h:508-570).  The result shares S's index tensors."""
    M, n_cols, K, a, b = _sddmm_dense_args(S_shape, A_shape, A_values, B_shape, B_values)
    if len(S_mode_indices) != 2 or len(S_mode_indices[0]) != 1 or len(S_mode_indices[1]) != 1:
        raise ValueError("scorch_ops_hip: S is not a coordinate (\"o,o\") operand")
    row = _index(S_mode_indices[0][0], "S rows")
    col = _index(S_mode_indices[1][0], "S cols")
    s_val = _flat(S_values, torch.float32, "S values")
    if row.numel() != s_val.numel() or col.numel() != s_val.numel():
        raise ValueError("scorch_ops_hip: S index and value lengths differ")
    dev = _device_of(row, col, s_val, a, b)
    out = _empty_like(s_val)
    L = native.lib()
    with _on_device(dev):
        stream = _stream(dev)
        pos = _coo_mask_row_ptr(row, col, M, n_cols, K)
        bl = _blocked(csr_plan(pos, col, M, n_cols, "S"), pos, col, M, n_cols, K) if pos is not None else None
        if bl is not None:
            # a mask made of 64 x 64 blocks, its coordinates in row-major order: the block kernel
            # writes the values in that same order
            rc = _blocked_sddmm(L, bl, 1, M, n_cols, K, s_val.numel(), s_val, a, b, out, None, stream)
        else:
            rc = L.scorch_hip_sddmm_coo_f32(M, n_cols, K, s_val.numel(), row.data_ptr(), col.data_ptr(),
                                            _mask_values_pointer(s_val), a.data_ptr(), b.data_ptr(), out.data_ptr(),
                                            stream)
    native.check(rc)
    return Tensor(out, S_mode_indices)


def _result_rows(plan: Optional[CsrPlan], crd: torch.Tensor):
    """The tensor of row coordinates for an SDDMM result over a CSR mask, and the pointer the
    kernel is to write them through (None: nothing to write).  The coordinates depend on the
    mask's pattern only: the first product with a planned mask writes them, later ones hand out
    the same tensor -- as the reference hands out a coordinate mask's own index tensors
    (src/scorch/ops.py:416-423) -- so a result's index tensors are not for writing to."""
    if plan is not None and plan.rows is not None:
        return plan.rows, None
    rows = _empty_like(crd)
    if plan is not None and not torch.cuda.is_current_stream_capturing():
        plan.rows = rows
    return rows, rows.data_ptr()


def sddmm_csr_float(result_shape, S_shape, S_mode_indices, S_values, A_shape, A_mode_indices, A_values,
                    B_shape, B_mode_indices, B_values):
    """SDDMM with a CSR mask.  The result is in coordinate format, one entry per
    mask entry in mask order: what the reference's generated kernel returns for
    this case (src/scorch/ops.py:638-666).  mode_indices = [[rows], [S's crd]]."""
    M, n_cols, K, a, b = _sddmm_dense_args(S_shape, A_shape, A_values, B_shape, B_values)
    pos, crd = _csr_parts(S_mode_indices, "S")
    s_val = _flat(S_values, torch.float32, "S values")
    if pos.numel() != M + 1 or crd.numel() != s_val.numel():
        raise ValueError("scorch_ops_hip: S array lengths do not match its shape")
    dev = _device_of(pos, crd, s_val, a, b)
    plan = csr_plan(pos, crd, M, n_cols, "S")
    out = _empty_like(s_val)
    rows, rows_ptr = _result_rows(plan, crd)
    L = native.lib()
    with _on_device(dev):
        stream = _stream(dev)
        bl = _blocked(plan, pos, crd, M, n_cols, K)
        lists = _sddmm_lists(plan, pos, crd, M, n_cols, K, L, stream) if bl is None else None
        if bl is not None:
            rc = _blocked_sddmm(L, bl, 1, M, n_cols, K, s_val.numel(), s_val, a, b, out, rows_ptr, stream)
        elif lists is not None:
            mask_ptr, listed_ptr = _listed_mask_values(s_val, lists, L, stream)
            rc = L.scorch_hip_sddmm_csr_listed_f32(1, M, n_cols, K, s_val.numel(), lists.data_ptr(), lists.numel(),
                                                   mask_ptr, listed_ptr, a.data_ptr(), b.data_ptr(),
                                                   out.data_ptr(), rows_ptr, stream)
        else:
            rc = L.scorch_hip_sddmm_csr_f32(M, n_cols, K, s_val.numel(), pos.data_ptr(), crd.data_ptr(),
                                            _mask_values_pointer(s_val), a.data_ptr(), b.data_ptr(), out.data_ptr(),
                                            rows_ptr, stream)
    native.check(rc)
    return Tensor(out, [[rows], [crd]])


# ---- neighbours of the path ---------------------------------------------------------
SOFTMAX_SHORT_ROW = 4096     # rows up to this length never reach the row softmax's giant-row pass


def _known_longest_row(pos: torch.Tensor, n_rows: int, nnz: int) -> Optional[int]:
    """The longest row of the pattern if a plan made for this row pointer says so (a product with
    the same pattern has inspected it), else None."""
    plan = getattr(pos, "_scorch_plan", None)
    if plan is not None and plan.key[0] == _stamp(pos) and plan.key[1][3] == nnz and plan.key[2] == n_rows:
        return plan.max_row
    return None


def _launch_softmax(L, dev, pos, batch: int, nnz: int, v, scale: float, out) -> None:
    """The row softmax of `batch` value arrays over one pattern; with the pattern's longest row known,
    the entry point that leaves out the launches no row of that length needs."""
    M = pos.numel() - 1
    longest = _known_longest_row(pos, M, nnz)
    with _on_device(dev):
        stream = _stream(dev)
        need = 0 if longest is not None and longest <= SOFTMAX_SHORT_ROW else \
            L.scorch_hip_softmax_csr_workspace_bytes(M, nnz)
        ws = _workspace(dev, stream, need) if need else None
        ws_ptr, ws_bytes = (ws.data_ptr(), ws.numel()) if need else (None, 0)
        if longest is not None:
            rc = L.scorch_hip_softmax_csr_known_rows_f32(batch, M, nnz, longest, pos.data_ptr(), v.data_ptr(),
                                                         float(scale), out.data_ptr(), ws_ptr, ws_bytes, stream)
        else:
            rc = L.scorch_hip_softmax_csr_batched_f32(batch, M, nnz, pos.data_ptr(), v.data_ptr(), float(scale),
                                                      out.data_ptr(), ws_ptr, ws_bytes, stream)
    native.check(rc)


def softmax_csr_float(row_ptr: torch.Tensor, values: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """Row softmax of ``scale * values`` over a CSR pattern
    (reference: bench/bench_sparse_transformer.py:277-297)."""
    pos = _index(row_ptr, "row_ptr")
    v = _flat(values, torch.float32, "values")
    dev = _device_of(pos, v)
    out = _empty_like(v)
    L = native.lib()
    _launch_softmax(L, dev, pos, 1, v.numel(), v, scale, out)
    return out


def csr_row_indices(row_ptr: torch.Tensor, nnz: int) -> torch.Tensor:
    """Row of every stored entry of a CSR pattern (int32[nnz])."""
    pos = _index(row_ptr, "row_ptr")
    dev = _device_of(pos)
    rows = _empty(nnz, dtype=torch.int32, device=dev)
    with _on_device(dev):
        rc = native.lib().scorch_hip_csr_row_indices(pos.numel() - 1, nnz, pos.data_ptr(),
                                                     rows.data_ptr(), _stream(dev))
    native.check(rc)
    return rows


def coo_row_ptr(row_idx: torch.Tensor, n_rows: int) -> Optional[torch.Tensor]:
    """CSR row pointer (int32[n_rows + 1]) of coordinates sorted by row, or None
    if they are not sorted or lie outside [0, n_rows).  One host read of a flag."""
    rows = _index(row_idx, "row coordinates")
    dev = _device_of(rows)
    pos = _empty(n_rows + 1, dtype=torch.int32, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    with _on_device(dev):
        rc = native.lib().scorch_hip_coo_row_ptr(n_rows, rows.numel(), rows.data_ptr(), pos.data_ptr(),
                                                 flag.data_ptr(), _stream(dev))
    native.check(rc)
    return None if int(flag.item()) else pos


def _coo_as_csr(mode_indices, values, n_rows: int, what: str):
    """(pos, crd, values) of a coordinate ("o,o") operand in row order.  Entries
    already grouped by ascending row (what STensor produces) are used as they
    are; anything else is first sorted by row, keeping the order inside a row."""
    if len(mode_indices) != 2 or len(mode_indices[0]) != 1 or len(mode_indices[1]) != 1:
        raise ValueError(f"scorch_ops_hip: {what} is not a coordinate (\"o,o\") operand")
    rows, cols = _index(mode_indices[0][0], what + " rows"), _index(mode_indices[1][0], what + " columns")
    if rows.numel() != cols.numel() or rows.numel() != values.numel():
        raise ValueError(f"scorch_ops_hip: {what}: coordinate and value arrays differ in length")
    pos = coo_row_ptr(rows, n_rows)
    if pos is None:
        if rows.numel() and (int(rows.min()) < 0 or int(rows.max()) >= n_rows):
            raise ValueError(f"scorch_ops_hip: {what} has a row coordinate outside [0, {n_rows})")
        rows, order = torch.sort(rows, stable=True)
        cols, values = cols[order].contiguous(), values[order].contiguous()
        pos = coo_row_ptr(rows, n_rows)
    return pos, cols, values


def spmm_coo_float(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values):
    """C = A @ B for A in coordinate form, fp32, dense result; repeated
    coordinates add up (reference: csrc/spmm.h:247-372).  The coordinates are
    turned into a row pointer on the device and the CSR kernel does the rest."""
    a_val = _flat(A_values, torch.float32, "A values")
    pos, crd, a_val = _coo_as_csr(A_mode_indices, a_val, int(A_shape[0]), "A")
    return _spmm(torch.float32, result_shape, A_shape, [[], [pos, crd]], a_val, B_shape, B_mode_indices,
                 B_values)


def spmspm_coo_float(result_shape, A_shape, A_mode_indices, A_values, B_shape, B_mode_indices, B_values):
    """C = A @ B, all in coordinate form, fp32 (reference: csrc/kernels.h:397-497):
    the result lists every structurally non-zero (row, column) once, rows
    ascending and columns ascending inside a row, sums that cancel included.
    Runs the CSR kernels between two index conversions on the device.  Where
    the reference emits one group of entries per run of equal rows in A, rows
    that are not grouped in A are merged here."""
    a_val = _flat(A_values, torch.float32, "A values")
    b_val = _flat(B_values, torch.float32, "B values")
    a_pos, a_crd, a_val = _coo_as_csr(A_mode_indices, a_val, int(A_shape[0]), "A")
    b_pos, b_crd, b_val = _coo_as_csr(B_mode_indices, b_val, int(B_shape[0]), "B")
    out = prebuilt_spmspm_csr_f32(result_shape, A_shape, [[], [a_pos, a_crd]], a_val, B_shape,
                                  [[], [b_pos, b_crd]], b_val)
    c_pos, c_crd = out.storage.index.mode_indices[1]
    rows = csr_row_indices(c_pos, int(c_crd.numel()))
    return Tensor(out.storage.value, [[rows], [c_crd]])


# ---- one pattern, several value arrays (one per attention head) ------------------------
def _batched_dense(t: torch.Tensor, batch: int, rows: int, cols: int, what: str) -> torch.Tensor:
    if t.dtype != torch.float32 or t.dim() != 3 or tuple(t.shape) != (batch, rows, cols):
        raise ValueError(f"scorch_ops_hip: {what} must be a float32 tensor of shape ({batch}, {rows}, {cols}), "
                         f"got {t.dtype} {tuple(t.shape)}")
    return t if t.is_contiguous() else t.contiguous()


def sddmm_csr_float_batched(S_shape, S_mode_indices, S_values, A: torch.Tensor, B: torch.Tensor):
    """out[h, p] = S.val[p] * <A[h, i_p, :], B[h, j_p, :]> for every head h and stored entry p of
    the CSR mask S: the SDDMM step of the reference's sparse attention for all heads in one launch
    (bench/bench_sparse_transformer.py:354-361 runs it per head).  A is (H, M, K), B is (H, n_cols, K).
    S_values may be None: every stored entry of the mask is 1 (no kernel reads anything for them).
    Returns (values of shape (H, nnz), row coordinates int32[nnz])."""
    M, n_cols = int(S_shape[0]), int(S_shape[1])
    pos, crd = _csr_parts(S_mode_indices, "S")
    s_val = _flat(S_values, torch.float32, "S values") if S_values is not None else None
    H, K = int(A.shape[0]), int(A.shape[2])
    a, b = _batched_dense(A, H, M, K, "A"), _batched_dense(B, H, n_cols, K, "B")
    nnz = crd.numel()
    if pos.numel() != M + 1 or (s_val is not None and nnz != s_val.numel()):
        raise ValueError("scorch_ops_hip: S array lengths do not match its shape")
    dev = _device_of(pos, crd, a, b) if s_val is None else _device_of(pos, crd, s_val, a, b)
    plan = csr_plan(pos, crd, M, n_cols, "S")
    out = _empty((H, nnz), dtype=torch.float32, device=dev)
    rows, rows_ptr = _result_rows(plan, crd)
    L = native.lib()
    with _on_device(dev):
        stream = _stream(dev)
        bl = _blocked(plan, pos, crd, M, n_cols, K) if H > 0 else None
        lists = _sddmm_lists(plan, pos, crd, M, n_cols, K, L, stream) if bl is None else None
        if bl is not None:
            rc = _blocked_sddmm(L, bl, H, M, n_cols, K, nnz, s_val, a, b, out, rows_ptr, stream)
        elif lists is not None:
            mask_ptr, listed_ptr = _listed_mask_values(s_val, lists, L, stream)
            rc = L.scorch_hip_sddmm_csr_listed_f32(H, M, n_cols, K, nnz, lists.data_ptr(), lists.numel(),
                                                   mask_ptr, listed_ptr, a.data_ptr(), b.data_ptr(),
                                                   out.data_ptr(), rows_ptr, stream)
        else:
            rc = L.scorch_hip_sddmm_csr_batched_f32(H, M, n_cols, K, nnz, pos.data_ptr(), crd.data_ptr(),
                                                    _mask_values_pointer(s_val), a.data_ptr(), b.data_ptr(),
                                                    out.data_ptr(), rows_ptr, stream)
    native.check(rc)
    return out, rows


def softmax_csr_float_batched(row_ptr: torch.Tensor, values: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """Row softmax of ``scale * values[h]`` over one CSR pattern for every head h;
    values is (H, nnz)."""
    pos = _index(row_ptr, "row_ptr")
    if values.dtype != torch.float32 or values.dim() != 2:
        raise ValueError("scorch_ops_hip: values must be a float32 tensor of shape (H, nnz)")
    v = values if values.is_contiguous() else values.contiguous()
    dev = _device_of(pos, v)
    H, nnz = int(v.shape[0]), int(v.shape[1])
    out = _empty_like(v)
    L = native.lib()
    _launch_softmax(L, dev, pos, H, nnz, v, scale, out)
    return out


def spmm_csr_float_batched(A_shape, A_mode_indices, A_values: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """C[h] = A_h @ B[h] where every A_h has the CSR pattern given and the values A_values[h]:
    the last step of the reference's sparse attention (bench/bench_sparse_transformer.py:370-372) for
    all heads in one launch.  A_values is (H, nnz), B is (H, K, N); returns (H, M, N)."""
    M, K = int(A_shape[0]), int(A_shape[1])
    pos, crd = _csr_parts(A_mode_indices, "A")
    if A_values.dtype != torch.float32 or A_values.dim() != 2:
        raise ValueError("scorch_ops_hip: A values must be a float32 tensor of shape (H, nnz)")
    a_val = A_values if A_values.is_contiguous() else A_values.contiguous()
    H, nnz = int(a_val.shape[0]), int(a_val.shape[1])
    N = int(B.shape[2])
    b = _batched_dense(B, H, K, N, "B")
    if pos.numel() != M + 1 or crd.numel() != nnz:
        raise ValueError("scorch_ops_hip: array lengths do not match the shapes")
    dev = _device_of(pos, crd, a_val, b)
    plan = csr_plan(pos, crd, M, K, "A")
    out = _empty((H, M, N), dtype=torch.float32, device=dev)
    if H == 0 or M == 0 or N == 0:
        return out
    L = native.lib()
    with _on_device(dev):
        stream = _stream(dev)
        bl = _blocked(plan, pos, crd, M, K, N) if SPMM_PATH == "auto" else None
        if bl is not None:
            rc = _blocked_spmm(L, bl, H, M, K, N, nnz, a_val, b, out, stream)
        elif SPMM_PATH == "rows" or (SPMM_PATH == "auto" and plan is not None and plan.max_row <= ROWS_KERNEL_MAX_ROW):
            rc = L.scorch_hip_spmm_csr_rows_batched_f32(H, M, K, N, nnz, pos.data_ptr(), crd.data_ptr(),
                                                        a_val.data_ptr(), b.data_ptr(), out.data_ptr(), stream)
        else:
            ws = _workspace(dev, stream, L.scorch_hip_spmm_csr_batched_workspace_bytes(H, M, nnz, N))
            bounds = _chunk_bounds(plan, pos, M, nnz, N, 4, L, stream) \
                if plan is not None and SPMM_PATH != "merge_unplanned" else None
            rc = L.scorch_hip_spmm_csr_batched_f32(H, M, K, N, nnz, pos.data_ptr(), crd.data_ptr(), a_val.data_ptr(),
                                                   b.data_ptr(), out.data_ptr(),
                                                   bounds.data_ptr() if bounds is not None else None,
                                                   bounds.numel() if bounds is not None else 0, ws.data_ptr(),
                                                   ws.numel(), stream)
    native.check(rc)
    return out


def sparse_attention_csr(row_ptr: torch.Tensor, col_idx: torch.Tensor, q: torch.Tensor, k: torch.Tensor,
                         v: torch.Tensor, scale: float) -> torch.Tensor:
    """softmax(scale * q k^T restricted to a CSR mask) v for q, k, v of shape (H, S, D), fp32: the
    reference's sparse attention (bench/bench_sparse_transformer.py:354-372: SDDMM, row softmax and
    SpMM per head) as three launches for all heads.  Any mask, any head dimension; rows of the mask
    without entries give zero rows."""
    H, S, D = (int(x) for x in q.shape)
    mask = [[], [row_ptr, col_idx]]
    scores, _ = sddmm_csr_float_batched([S, S], mask, None, q, k)
    probs = softmax_csr_float_batched(row_ptr, scores, scale)
    return spmm_csr_float_batched([S, S], mask, probs, v)


class BlockMask:
    """A CSR attention mask regrouped into 64 x 64 blocks for the fused attention kernel: the block
    pattern in CSR form, and for every active block either -1 (all 4096 entries live) or the index
    of its 64-word bit mask (bit j of word r: query r of the block row attends to key j of the
    block).  Blocks with equal masks share one."""
    __slots__ = ("S", "block", "block_row_ptr", "block_col_idx", "block_mask_index", "block_masks", "nnz",
                 "items", "split_rows", "n_slots", "schedule32", "block_row_lens", "pairing")

    def __init__(self, S, block, block_row_ptr, block_col_idx, block_mask_index, block_masks, nnz):
        self.S, self.block, self.nnz = S, block, nnz
        self.block_row_ptr, self.block_col_idx = block_row_ptr, block_col_idx
        self.block_mask_index, self.block_masks = block_mask_index, block_masks
        # set by split_long_block_rows when some block row is shared out among workgroups
        self.items = self.split_rows = None
        self.n_slots = 0
        self.schedule32 = None      # the fp32 kernel's own sharing-out (see _fp32_schedule)
        self.block_row_lens = None  # active blocks per block row, on the host (numpy), once it has been read
        self.pairing = {}           # (item list, heads, head dimension) -> (workgroups take two items?, priority step)

    def row_lens(self):
        """Active blocks per block row as a numpy array on the host (read from the device once)."""
        if self.block_row_lens is None:
            import numpy as np
            brp = self.block_row_ptr.cpu().numpy().astype(np.int64)
            self.block_row_lens = brp[1:] - brp[:-1]
        return self.block_row_lens

    @property
    def n_active_blocks(self) -> int:
        return int(self.block_col_idx.numel())

    @property
    def n_masks(self) -> int:
        return int(self.block_masks.numel()) // self.block

    @property
    def density_in_blocks(self) -> float:
        """Share of the entries of the active blocks that are live: the fused kernel computes whole
        blocks, so 1 / this is its overhead over the mask's own entry count."""
        return self.nnz / max(1, self.n_active_blocks * self.block * self.block)


def block_mask_from_csr(row_ptr: torch.Tensor, col_idx: torch.Tensor, S: int) -> BlockMask:
    """Regroup an S x S CSR mask (S a multiple of 64) on a HIP device into a BlockMask: the two
    kernel passes of _describe_blocks over the entries, then the blocks that are not fully stored
    are compared with one another so that equal masks are kept once.  Done once per mask (see
    attention_block_mask for the cached form); repeated entries and unsorted rows are tolerated."""
    block = 64
    if S % block:
        raise ValueError("scorch_ops_hip: S must be a multiple of 64")
    pos, crd = _index(row_ptr, "row_ptr"), _index(col_idx, "col_idx")
    dev = _device_of(pos, crd)
    if pos.numel() != S + 1:
        raise ValueError("scorch_ops_hip: row_ptr length does not match S")
    csr_plan(pos, crd, S, S, "mask")                      # validates the index (ValueError), once per tensor pair
    nb = S // block
    brp, arrays = _describe_blocks(pos, crd, S, S)
    if arrays is None:                                    # no entries at all
        empty = lambda dtype: torch.zeros(0, dtype=dtype, device=dev)
        bm = BlockMask(S, block, torch.zeros(nb + 1, dtype=torch.int32, device=dev), empty(torch.int32),
                       empty(torch.int32), empty(torch.int64), 0)
        bm.block_row_lens = brp[1:] - brp[:-1]
        return bm
    stored = arrays["block_nnz"]
    n_active = int(stored.numel())
    mask_index = torch.full((n_active,), -1, dtype=torch.int32, device=dev)
    partial = torch.nonzero(stored != block * block).flatten()
    if partial.numel():
        masks, which = torch.unique(arrays["block_words"].view(n_active, block)[partial], dim=0, return_inverse=True)
        mask_index[partial] = which.to(torch.int32)
    else:
        masks = torch.zeros((0, block), dtype=torch.int64, device=dev)
    bm = BlockMask(S, block, arrays["block_row_ptr"], arrays["block_col_idx"], mask_index,
                   masks.contiguous().view(-1), int(stored.sum()))
    bm.block_row_lens = brp[1:] - brp[:-1]
    return bm


# workgroups of the fused bf16 attention kernel a CU holds at once, by head dimension
ATTENTION_WORKGROUPS_PER_CU = {32: 6, 64: 4, 128: 2}


_cu_counts: Dict[int, int] = {}


def _cu_count(device) -> int:
    index = torch.device(device).index or 0
    if index not in _cu_counts:
        _cu_counts[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _cu_counts[index]


def pair_attention_items(lens, heads: int, D: int, n_cus: int = 256) -> bool:
    """Whether the fused bf16 attention kernel should give every workgroup two work items, the
    k-th longest and then the k-th shortest (scorch_hip_attn_blocksparse_split_bf16, pair_items).
    `lens`: key blocks per item.  Pairing evens the workgroups out and halves their number; it
    pays where the items differ in length, or are so short that a workgroup's start and end
    weigh, and the launch is between about 0.6 and 4 times what the chip holds at once, and costs
    elsewhere (S = 8192, 16 heads, D = 64, measured: the benchmark's causal strided mask -7 %,
    four blocks in every row -9 %, twelve +1 %; a causal mask at S = 4096 -15 % with 16 heads,
    +7 % with 4, -3 % with 128; at S = 16384 with D = 128 +3 %)."""
    import numpy as np
    lens = np.asarray(lens)
    if lens.size < 2 or D not in ATTENTION_WORKGROUPS_PER_CU:
        return False
    slots = n_cus * ATTENTION_WORKGROUPS_PER_CU[D]
    rounds = lens.size * heads / slots
    mean = float(lens.mean())
    uneven = float(lens.max()) > 1.25 * mean
    return 0.6 <= rounds <= 4.0 and mean <= 64 and (uneven or mean <= 6)


def attention_priority_step(lens, heads: int, D: int, pair: bool, n_cus: int = 256) -> int:
    """The priority_step to hand scorch_hip_attn_blocksparse_split_bf16 for work items of `lens` key
    blocks (0: leave the wavefronts' priorities alone).  With a step a wavefront's priority follows
    what its workgroup has left to do, in four levels: a quarter of the most any workgroup gets.
    It pays where a CU holds two workgroups or more at a time and the launch is short of four
    times what the chip holds at once (measured at S = 8192, 16 heads, D = 64, on top of the
    pairing decision: the benchmark's causal strided mask -4 to -5 %, four, twelve and twenty
    blocks in every row -3 %, a dense mask -3 %; causal masks at S = 4096 0 to -2 %) and is left
    out elsewhere (a causal mask with 4 heads, one workgroup per CU: +4 %; 64 heads with four
    blocks in every row, eight rounds: +3 %; S = 16,384 with D = 128, four rounds: +1 %)."""
    import numpy as np
    lens = np.asarray(lens)
    if lens.size == 0 or D not in ATTENTION_WORKGROUPS_PER_CU:
        return 0
    workgroups = ((lens.size + 1) // 2 if pair else lens.size) * heads
    if workgroups < 2 * n_cus or workgroups >= 4 * n_cus * ATTENTION_WORKGROUPS_PER_CU[D]:
        return 0            # one workgroup per CU: nothing to arbitrate; four rounds and more: nothing measurable
    if pair:
        ordered = np.sort(lens)[::-1]
        half = (lens.size + 1) // 2
        second = ordered[::-1][:half].copy()
        if lens.size % 2:
            second[-1] = 0                      # the middle item has no partner
        most = int((ordered[:half] + second).max())
    else:
        most = int(lens.max())
    return max(1, -(-most // 4))


def split_long_block_rows(bm: BlockMask, longest: Optional[int] = None, list_unequal_rows: bool = False) -> BlockMask:
    """Share block rows with more than `longest` key blocks out among several workgroups (in
    stretches of equal length up to `longest`); by default `longest` is twice the mean number of
    key blocks per block row, at least 8, so that masks whose rows are of similar length are left
    alone and a row that attends to everything (a global token) is not the one workgroup the whole
    launch waits for.  Fills bm.items / bm.split_rows / bm.n_slots (None / None / 0 when no row is
    long enough -- unless `list_unequal_rows` asks for the rows, longest first, whenever they differ
    in length)."""
    lens = bm.row_lens()
    nb = int(lens.size)
    if longest is None:
        longest = max(8, 2 * -(-int(lens.sum()) // max(nb, 1)))
    bm.items = bm.split_rows = None
    bm.n_slots = 0
    most = int(lens.max()) if nb else 0
    if longest < 1 or most <= longest:
        if not (list_unequal_rows and nb and int(lens.min()) != most):
            return bm
    items, split_rows, n_slots = _stretches(lens, longest if longest >= 1 else max(most, 1), True)
    dev = bm.block_row_ptr.device
    bm.items = torch.from_numpy(items).to(dev).reshape(-1)
    bm.split_rows = torch.from_numpy(split_rows).to(dev).reshape(-1)
    bm.n_slots = n_slots
    return bm


def attention_block_mask(row_ptr: torch.Tensor, col_idx: torch.Tensor, S: int) -> BlockMask:
    """block_mask_from_csr, kept with the mask's row_ptr tensor and rebuilt when either index
    array is replaced or written to."""
    key = (_stamp(row_ptr), _stamp(col_idx), S)
    cached = getattr(row_ptr, "_scorch_block_mask", None)
    if cached is not None and cached[0] == key and _same(cached[2], col_idx):
        return cached[1]
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("scorch_ops_hip: the block form of an attention mask is built with host reads; call "
                           "attention_block_mask(row_ptr, col_idx, S) once before capturing")
    bm = split_long_block_rows(block_mask_from_csr(row_ptr, col_idx, S))
    try:
        row_ptr._scorch_block_mask = (key, bm, weakref.ref(col_idx))
    except AttributeError:
        pass
    return bm


def sparse_attention_bf16(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, row_ptr: torch.Tensor,
                          col_idx: torch.Tensor, scale: float) -> torch.Tensor:
    """softmax(scale * q k^T restricted to a CSR mask) v for bf16 q, k, v of shape (H, S, D), D in
    {32, 64, 128}, S a multiple of 64, in one fused kernel: the mask is regrouped into 64 x 64
    blocks with bit masks once (attention_block_mask) and the kernel computes every block that
    holds an entry.  Same result as sparse_attention_csr up to bf16 rounding of the operands, the
    probabilities and the result."""
    bm = attention_block_mask(row_ptr, col_idx, int(q.shape[1]))
    if bm.items is None:
        return attn_blocksparse_bf16(q, k, v, bm.block_row_ptr, bm.block_col_idx, scale, block=bm.block,
                                     block_mask_index=bm.block_mask_index, block_masks=bm.block_masks)
    return attn_blocksparse_split_bf16(q, k, v, bm, scale)


def sparse_attention_f32(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, row_ptr: torch.Tensor,
                         col_idx: torch.Tensor, scale: float) -> torch.Tensor:
    """softmax(scale * q k^T restricted to a CSR mask) v for fp32 q, k, v of shape (H, S, D), D in
    {32, 64, 128}, S a multiple of 64, in one fused kernel with fp32 probabilities and sums: what
    sparse_attention_csr computes in three launches (the reference's per-head composition,
    bench/bench_sparse_transformer.py:354-372), to fp32 rounding.  The kernel computes every
    64 x 64 block that holds an entry, so it pays for masks that fill their blocks reasonably."""
    return attn_blocksparse_f32(q, k, v, attention_block_mask(row_ptr, col_idx, int(q.shape[1])), scale)


FP32_ATTENTION_STRETCH = 16


def _fp32_schedule(bm: BlockMask):
    """(items, split_rows, n_slots) for the fp32 attention kernel, kept with the BlockMask.  Its
    key blocks take six times as long as the bf16 kernel's, so what a stretch's partial results
    cost matters little and an even load matters much: where block rows differ in length by more
    than a quarter of the mean they go out in stretches of at most 16 key blocks (and at most
    twice the mean, at least 8), longest first (a causal mask at S = 4096: a quarter less time);
    rows of similar length stay whole.  Under stream capture a BlockMask that has no schedule yet
    is served by whole rows."""
    if bm.schedule32 is None:
        if bm.block_row_ptr.is_cuda and torch.cuda.is_current_stream_capturing():
            return None, None, 0
        plain = BlockMask(bm.S, bm.block, bm.block_row_ptr, bm.block_col_idx, None, None, bm.nnz)
        lens = bm.row_lens()
        plain.block_row_lens = lens
        mean = float(lens.sum()) / max(int(lens.size), 1)
        longest = int(lens.max()) if lens.size else 0
        if longest > 1.25 * mean:      # (rows of similar length are best left whole)
            longest = min(FP32_ATTENTION_STRETCH, max(8, 2 * math.ceil(mean)))
        split_long_block_rows(plain, longest, list_unequal_rows=True)
        bm.schedule32 = (plain.items, plain.split_rows, plain.n_slots)
    return bm.schedule32


def attn_blocksparse_f32(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, bm: BlockMask, scale: float) -> torch.Tensor:
    """The fp32 fused attention kernel over a BlockMask (block_mask_index / block_masks may be None:
    every listed block fully live; rows that split_long_block_rows shared out go through a
    workspace and a second kernel)."""
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.dtype != torch.float32 or t.dim() != 3:
            raise TypeError(f"scorch_ops_hip: {name} must be a float32 tensor of shape (H, S, D)")
    if q.shape != k.shape or q.shape != v.shape:
        raise ValueError("scorch_ops_hip: q, k and v must have the same shape")
    q, k, v = (t if t.is_contiguous() else t.contiguous() for t in (q, k, v))
    index_tensors = [t for t in (bm.block_row_ptr, bm.block_col_idx, bm.block_mask_index, bm.block_masks)
                     if t is not None]
    dev = _device_of(q, k, v, *index_tensors)
    H, S, D = q.shape
    if S != bm.S:
        raise ValueError("scorch_ops_hip: the BlockMask was built for another sequence length")
    ptr = lambda t: t.data_ptr() if t is not None and t.numel() else None
    items, split_rows, n_slots = _fp32_schedule(bm)
    n_items = items.numel() // 4 if items is not None else 0
    n_split = split_rows.numel() // 4 if split_rows is not None else 0
    out = _empty_like(q)
    L = native.lib()
    with _on_device(dev):
        stream = _stream(dev)
        need = L.scorch_hip_attn_blocksparse_f32_workspace_bytes(H, n_slots, D) if n_items else 0
        ws = _workspace(dev, stream, need) if need else None
        rc = L.scorch_hip_attn_blocksparse_f32(
            H, S, D, bm.block, bm.n_active_blocks, ptr(bm.block_row_ptr), ptr(bm.block_col_idx),
            ptr(bm.block_mask_index), bm.n_masks if bm.block_masks is not None else 0, ptr(bm.block_masks),
            n_items, ptr(items), n_split, ptr(split_rows), n_slots if n_items else 0,
            q.data_ptr(), k.data_ptr(), v.data_ptr(), float(scale), out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, stream)
    native.check(rc)
    if ws is not None:
        out._scorch_workspace = ws     # a buffer handed out during a graph capture lives as long as the result
    return out


def _attn_bf16_args(q, k, v):
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.dtype != torch.bfloat16 or t.dim() != 3:
            raise TypeError(f"scorch_ops_hip: {name} must be a bfloat16 tensor of shape (H, S, D)")
    if q.shape != k.shape or q.shape != v.shape:
        raise ValueError("scorch_ops_hip: q, k and v must have the same shape")
    return tuple(t if t.is_contiguous() else t.contiguous() for t in (q, k, v))


def _attn_bf16_items(q, k, v, bm: BlockMask, items: torch.Tensor, split_rows: Optional[torch.Tensor], n_slots: int,
                     scale: float, pair: bool, priority_step: int = 0) -> torch.Tensor:
    """The fused bf16 kernel over a list of work items (scorch_hip_attn_blocksparse_split_bf16)."""
    tensors = [t for t in (bm.block_col_idx, bm.block_mask_index, bm.block_masks, items) if t is not None]
    dev = _device_of(q, k, v, *tensors)
    H, S, D = q.shape
    if S != bm.S:
        raise ValueError("scorch_ops_hip: the BlockMask was built for another sequence length")
    ptr = lambda t: t.data_ptr() if t is not None and t.numel() else None
    out = _empty_like(q)
    L = native.lib()
    with _on_device(dev):
        stream = _stream(dev)
        need = L.scorch_hip_attn_blocksparse_split_workspace_bytes(H, n_slots, D)
        ws = _workspace(dev, stream, need) if need else None
        rc = L.scorch_hip_attn_blocksparse_split_bf16(
            H, S, D, bm.block, bm.n_active_blocks, items.numel() // 4, items.data_ptr(), int(pair), int(priority_step),
            split_rows.numel() // 4 if split_rows is not None else 0, ptr(split_rows), n_slots,
            ptr(bm.block_col_idx), ptr(bm.block_mask_index) if bm.block_mask_index is not None else None,
            bm.n_masks if bm.block_masks is not None else 0, ptr(bm.block_masks), q.data_ptr(), k.data_ptr(),
            v.data_ptr(), float(scale), out.data_ptr(), ws.data_ptr() if ws is not None else None,
            ws.numel() if ws is not None else 0, stream)
    native.check(rc)
    if ws is not None:
        out._scorch_workspace = ws     # a buffer handed out during a graph capture lives as long as the result
    return out


# For measurements: SCORCH_HIP_ATTN_PAIRING=0 / SCORCH_HIP_ATTN_PRIORITY=0 keep one work item per
# workgroup / leave the wavefronts' priorities alone whatever the mask looks like.
ATTENTION_PAIRING = os.environ.get("SCORCH_HIP_ATTN_PAIRING", "1") not in ("", "0")
ATTENTION_PRIORITY = os.environ.get("SCORCH_HIP_ATTN_PRIORITY", "1") not in ("", "0")


def _launch_plan(lens, heads: int, D: int, device):
    """(pair the items?, priority step) for a list of work items of `lens` key blocks."""
    n_cus = _cu_count(device)
    pair = pair_attention_items(lens, heads, D, n_cus) if ATTENTION_PAIRING else False
    return pair, attention_priority_step(lens, heads, D, pair, n_cus) if ATTENTION_PRIORITY else 0


def _pairing(bm: BlockMask, kind: str, lens, heads: int, D: int, device):
    """_launch_plan for one of the BlockMask's item lists, remembered per (list, heads, D)."""
    key = (kind, int(heads), int(D))
    if key not in bm.pairing:
        bm.pairing[key] = _launch_plan(lens, int(heads), int(D), device)
    return bm.pairing[key]


def attn_blocksparse_split_bf16(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, bm: BlockMask,
                                scale: float) -> torch.Tensor:
    """attn_blocksparse_bf16 over a BlockMask whose long block rows split_long_block_rows has
    shared out among workgroups: their partial results go through a workspace and a second kernel
    combines them.  Same result up to the rounding of the partial sums' combination."""
    if bm.items is None:
        raise ValueError("scorch_ops_hip: this BlockMask has no shared-out rows (split_long_block_rows)")
    q, k, v = _attn_bf16_args(q, k, v)
    key = ("items", int(q.shape[0]), int(q.shape[2]))
    if key not in bm.pairing:
        if q.is_cuda and torch.cuda.is_current_stream_capturing():
            plan = (False, 0)                     # (deciding needs a host read of the items)
        else:
            rows = bm.items.view(-1, 4)
            plan = _pairing(bm, "items", (rows[:, 2] - rows[:, 1]).cpu().numpy(), q.shape[0], q.shape[2], q.device)
    else:
        plan = bm.pairing[key]
    return _attn_bf16_items(q, k, v, bm, bm.items, bm.split_rows, bm.n_slots, scale, plan[0], plan[1])


def _block_row_schedule(brp: torch.Tensor):
    """(key blocks per block row on the host, the block rows as work items longest first, pairing
    decisions) of a block row pointer, read back once and kept with the tensor; None while the
    stream is capturing and nothing is known yet."""
    import numpy as np
    cached = getattr(brp, "_scorch_rows", None)
    if cached is not None and cached[0] == _stamp(brp):
        return cached[1:]
    if torch.cuda.is_current_stream_capturing():
        return None
    ptrs = brp.cpu().numpy().astype(np.int64)
    lens = ptrs[1:] - ptrs[:-1]
    items, _, _ = _stretches(lens, max(int(lens.max()), 1) if lens.size else 1, True)
    entry = (_stamp(brp), lens, torch.from_numpy(items).to(brp.device).reshape(-1), {})
    try:
        brp._scorch_rows = entry
    except (AttributeError, RuntimeError):
        pass
    return entry[1:]


def attn_blocksparse_bf16(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, block_row_ptr: torch.Tensor,
                          block_col_idx: torch.Tensor, scale: float, block: int = 64,
                          block_mask_index: Optional[torch.Tensor] = None,
                          block_masks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """softmax(scale * q k^T over a block mask) v for q, k, v of shape (H, S, D),
    bf16, in one kernel; fp32 accumulation, bf16 result.  The fused form of the
    per-head SDDMM -> softmax -> SpMM pipeline of
    bench/bench_sparse_transformer.py:354-372.  With block_mask_index (int32 per active block, -1
    = fully live) and block_masks (int64, 64 words per mask) a block is restricted to the entries
    its bit mask names.  Where it pays (pair_attention_items, attention_priority_step) the block rows
    go to the kernel as a list of work items, of which every workgroup takes two and / or whose
    wavefronts' priorities follow the work they have left; the result is the same bit for bit."""
    q, k, v = _attn_bf16_args(q, k, v)
    brp, bci = _index(block_row_ptr, "block_row_ptr"), _index(block_col_idx, "block_col_idx")
    dev = _device_of(q, k, v, brp, bci)
    H, S, D = q.shape
    if brp.numel() != S // block + 1:
        raise ValueError("scorch_ops_hip: block_row_ptr length does not match S / block")
    bmi, n_masks = None, 0
    if block_mask_index is not None:
        bmi = _index(block_mask_index, "block_mask_index")
        if block_masks is None or block_masks.dtype != torch.int64 or not block_masks.is_contiguous():
            raise TypeError("scorch_ops_hip: block_masks must be a contiguous int64 tensor")
        if bmi.numel() != bci.numel():
            raise ValueError("scorch_ops_hip: block_mask_index must have one entry per active block")
        if block_masks.numel() % block or block_masks.device != q.device or bmi.device != q.device:
            raise ValueError("scorch_ops_hip: block_masks must hold 64 words per mask on the operands' device")
        n_masks = block_masks.numel() // block
        # the kernel trusts the mask indices as it trusts block_col_idx; a caller that built them by
        # hand gets them checked here, once per index tensor
        if getattr(bmi, "_scorch_mask_checked", None) != (_stamp(bmi), n_masks):
            if bmi.numel() and int(bmi.max()) >= n_masks:
                raise ValueError("scorch_ops_hip: block_mask_index names a mask beyond block_masks")
            try:
                bmi._scorch_mask_checked = (_stamp(bmi), n_masks)
            except AttributeError:
                pass
    schedule = _block_row_schedule(brp) if block == 64 and D in ATTENTION_WORKGROUPS_PER_CU else None
    if schedule is not None:
        lens, items, pairing = schedule
        key = (int(H), int(D))
        if key not in pairing:
            pairing[key] = _launch_plan(lens, int(H), int(D), dev)
        pair, priority_step = pairing[key]
        if pair or priority_step:
            rows = BlockMask(int(S), block, brp, bci, bmi, block_masks if bmi is not None else None, 0)
            return _attn_bf16_items(q, k, v, rows, items, None, 0, scale, pair, priority_step)
    out = _empty_like(q)
    with _on_device(dev):
        if bmi is None:
            rc = native.lib().scorch_hip_attn_blocksparse_bf16(H, S, D, block, bci.numel(), brp.data_ptr(),
                                                               bci.data_ptr(), q.data_ptr(), k.data_ptr(),
                                                               v.data_ptr(), float(scale), out.data_ptr(),
                                                               _stream(dev))
        else:
            rc = native.lib().scorch_hip_attn_blocksparse_masked_bf16(
                H, S, D, block, bci.numel(), brp.data_ptr(), bci.data_ptr(), bmi.data_ptr(), n_masks,
                block_masks.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), float(scale), out.data_ptr(),
                _stream(dev))
    native.check(rc)
    return out
