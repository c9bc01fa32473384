"""STensor: a tensor stored in a per-mode format (reference: src/scorch/stensor.py).

This is the part of the reference's tensor model that the prebuilt SpMM/SDDMM
path touches: construction from torch tensors (dense, CSR, COO), the
``values`` / ``index.mode_indices`` / ``shape`` / ``format`` accessors the
kernel dispatch reads, and conversion back to torch.  Unlike the reference,
whose ``to()`` is a stub (stensor.py:147-150), an STensor here can live on a
GPU: ``to(device)`` moves the value and index tensors.

Format conversion is done with torch's own sparse routines on whatever device
the tensor is on; the reference's JIT-compiled converters are not part of this
package.
"""
from __future__ import annotations

from typing import List, Optional, Tuple, Union

import torch

from .format import LevelFormat, LevelType, TensorFormat, parse_format
from .storage import TensorIndex, TensorStorage



def _sorted_unique_entries(rows: torch.Tensor, cols: torch.Tensor, values: torch.Tensor, n_cols: int):
    """Entries sorted by (row, col); values of repeated coordinates are summed."""
    if rows.numel() == 0:
        return rows, cols, values
    key = rows * int(n_cols) + cols
    key, order = torch.sort(key, stable=True)
    values = values[order]
    first = torch.ones_like(key, dtype=torch.bool)
    first[1:] = key[1:] != key[:-1]
    if not bool(first.all()):
        segment = torch.cumsum(first.to(torch.int64), dim=0) - 1
        summed = torch.zeros(int(segment[-1]) + 1, dtype=values.dtype, device=values.device)
        summed.index_add_(0, segment, values)
        key, values = key[first], summed
    return key // int(n_cols), key % int(n_cols), values


class STensor(torch.nn.Module):
    def __init__(self, name: Optional[str] = None, shape: Optional[Tuple[int, ...]] = None,
                 storage: Optional[TensorStorage] = None, index: Optional[TensorIndex] = None,
                 value: Optional[torch.Tensor] = None, requires_grad: Optional[bool] = False) -> None:
        super().__init__()
        # plain attributes (no parameter, buffer or sub-module among them): set past
        # nn.Module.__setattr__, whose type checks cost more than everything else here
        put = object.__setattr__
        put(self, "_storage", storage if storage is not None else TensorStorage(index=index, value=value,
                                                                                shape=shape))
        put(self, "_name", name)
        put(self, "_shape", tuple(shape) if shape is not None else None)
        if value is not None:
            put(self, "_dtype", value.dtype)
        elif storage is not None and storage._value is not None:
            put(self, "_dtype", storage._value.dtype)
        else:
            put(self, "_dtype", torch.float32)
        put(self, "requires_grad", requires_grad)

    # ---- accessors the dispatch reads ------------------------------------------
    @property
    def name(self) -> str:
        assert self._name is not None, "Tensor name is not set."
        return self._name

    @name.setter
    def name(self, name: str) -> None:
        self._name = name

    @property
    def storage(self) -> TensorStorage:
        assert self._storage is not None, "Tensor storage is not set."
        return self._storage

    @property
    def values(self) -> torch.Tensor:
        return self.storage.value

    @property
    def index(self) -> TensorIndex:
        return self.storage.index

    @property
    def has_index(self) -> bool:
        return self.storage.has_index

    @property
    def format(self) -> TensorFormat:
        fmt = self.index.format
        assert fmt is not None, "Tensor format is not set."
        return fmt

    @property
    def dtype(self) -> torch.dtype:
        return self._dtype

    @property
    def shape(self) -> Tuple[int, ...]:
        return self._shape if self._shape is not None else tuple()

    @property
    def device(self) -> torch.device:
        return self.values.device

    @property
    def is_cuda(self) -> bool:
        return self.values.is_cuda

    def dim(self) -> int:
        return len(self.shape)

    def _nnz(self) -> int:
        return self.values.numel()

    def __repr__(self) -> str:
        return "Tensor"

    # ---- residency ---------------------------------------------------------------
    def to(self, device) -> "STensor":
        """Copy of the tensor with values and indices on ``device``."""
        return STensor(name=self._name, shape=self.shape, storage=self.storage.to(device))

    def cuda(self) -> "STensor":
        return self.to(torch.device("cuda", torch.cuda.current_device()))

    def cpu(self) -> "STensor":
        return self.to(torch.device("cpu"))

    def copy(self) -> "STensor":
        return STensor(name=self._name, shape=self.shape, storage=self.storage.copy())

    clone = copy

    def validate(self) -> None:
        """Raise ValueError unless the index arrays describe a tensor of this shape: row
        pointers that start at 0, never decrease and end at the number of stored entries,
        coordinates inside the shape (the reference leaves this method unimplemented,
        stensor.py:142-145).  Reads the index arrays and synchronises."""
        fmt = str(self.format)
        count = self.values.numel()
        if self.format.is_dense():
            expected = 1
            for extent in self.shape:
                expected *= int(extent)
            if count != expected:
                raise ValueError(f"STensor: {count} values for a dense tensor of shape {tuple(self.shape)}")
            return
        if self.dim() != 2 or fmt not in ("d,s", "o,o"):
            raise NotImplementedError(f"STensor.validate for format {fmt!r}")
        order = self.index.mode_order
        extents = [int(self.shape[order[0]]), int(self.shape[order[1]])]    # of the stored modes
        levels = self.index.mode_indices
        if fmt == "d,s":
            pos, crd = levels[1]
            if pos.numel() != extents[0] + 1 or crd.numel() != count:
                raise ValueError("STensor: index array lengths do not match the shape and the values")
            rows_ok = bool(pos[0] == 0) and bool(pos[-1] == count) and bool((pos[1:] >= pos[:-1]).all())
            if not rows_ok:
                raise ValueError(f"STensor: row pointers must start at 0, never decrease and end at {count}")
            stored = [crd]
            limits = [extents[1]]
        else:
            stored = [levels[0][0], levels[1][0]]
            limits = extents
            if any(c.numel() != count for c in stored):
                raise ValueError("STensor: coordinate and value arrays differ in length")
        for coordinates, limit in zip(stored, limits):
            if count and (int(coordinates.min()) < 0 or int(coordinates.max()) >= limit):
                raise ValueError(f"STensor: a coordinate lies outside [0, {limit})")

    # ---- construction --------------------------------------------------------------
    @staticmethod
    def _csr(shape, crow, col, values, name, mode_order=None) -> "STensor":
        fmt = TensorFormat([LevelFormat(LevelType.DENSE), LevelFormat(LevelType.COMPRESSED)])
        return STensor(name=name, shape=tuple(shape), storage=TensorStorage(
            index=TensorIndex(fmt, [[], [crow, col]], mode_order=mode_order), value=values))

    @staticmethod
    def _coo(shape, indices, values, name, mode_order=None) -> "STensor":
        fmt = TensorFormat([LevelFormat(LevelType.COORDINATE) for _ in shape])
        return STensor(name=name, shape=tuple(shape), storage=TensorStorage(
            index=TensorIndex(fmt, [[indices[i]] for i in range(len(shape))], mode_order=mode_order),
            value=values))

    @staticmethod
    def from_csr(csr_matrix: torch.Tensor, name: Optional[str] = None) -> "STensor":
        """2-D torch CSR tensor -> "d,s" STensor sharing its arrays
        (reference: stensor.py:271-315)."""
        assert csr_matrix.is_sparse_csr, "Input tensor must be a sparse CSR tensor."
        assert csr_matrix.dim() == 2, "CSR format is only valid for 2D matrices."
        return STensor._csr(csr_matrix.shape, csr_matrix.crow_indices(), csr_matrix.col_indices(),
                            csr_matrix.values(), name or "tensor")

    @staticmethod
    def from_csr_arrays(row_ptr: torch.Tensor, col_idx: torch.Tensor, values: torch.Tensor,
                        shape: Tuple[int, int], name: Optional[str] = None) -> "STensor":
        """"d,s" STensor over caller-owned arrays (no torch sparse tensor in between)."""
        return STensor._csr(shape, row_ptr, col_idx, values, name or "tensor")

    @staticmethod
    def from_coo(coo_matrix: Optional[torch.Tensor] = None, indices: Optional[torch.Tensor] = None,
                 values: Optional[torch.Tensor] = None, shape: Optional[Tuple[int, ...]] = None,
                 name: Optional[str] = None) -> "STensor":
        """torch COO tensor (coalesced first) or raw (indices, values, shape) ->
        all-coordinate STensor (reference: stensor.py:318-365)."""
        if coo_matrix is not None:
            coo_matrix = coo_matrix.coalesce()
            indices, values, shape = coo_matrix.indices(), coo_matrix.values(), coo_matrix.shape
        assert indices is not None and values is not None and shape is not None
        return STensor._coo(tuple(shape), indices, values, name or "tensor")

    @staticmethod
    def from_torch(tensor: torch.Tensor, name: Optional[str] = None,
                   mode_order: Optional[List[int]] = None) -> "STensor":
        """torch tensor of any layout -> STensor (reference: stensor.py:368-452).
        Strided tensors become all-dense with ``values = tensor.flatten()``."""
        name = name or "tensor"
        if mode_order:
            tensor = tensor.permute(*mode_order)
        else:
            mode_order = list(range(tensor.dim()))
        if tensor.layout == torch.sparse_coo:
            tensor = tensor.coalesce()
            return STensor._coo(tensor.shape, tensor.indices(), tensor.values(), name, mode_order)
        if tensor.layout == torch.sparse_csr:
            return STensor._csr(tensor.shape, tensor.crow_indices(), tensor.col_indices(),
                                tensor.values(), name, mode_order)
        fmt = TensorFormat([LevelFormat(LevelType.DENSE) for _ in tensor.shape])
        value = tensor.flatten()
        if value is not tensor and value.is_cuda and value.data_ptr() == tensor.data_ptr():
            # a view of the caller's tensor: layouts the device kernels cache for this
            # operand are kept on the caller's object, which outlives the view
            value._scorch_origin = tensor
        return STensor(name=name, shape=tuple(tensor.shape), storage=TensorStorage(
            index=TensorIndex(fmt, [[] for _ in tensor.shape], mode_order=mode_order),
            value=value))

    # ---- conversion ------------------------------------------------------------------
    def _as_torch_sparse(self) -> torch.Tensor:
        kinds = [t.value for t in self.format.get_level_types()]
        idx = self.index.mode_indices
        if kinds == ["d", "s"]:
            return torch.sparse_csr_tensor(idx[1][0], idx[1][1], self.values, size=self.shape)
        if all(k == "o" for k in kinds):
            coords = torch.stack([level[0].to(torch.int64) for level in idx], dim=0)
            return torch.sparse_coo_tensor(coords, self.values, size=self.shape)
        raise NotImplementedError(f"no torch layout for format {self.format}")

    def to_dense(self, fmt=None, in_place: bool = False) -> "STensor":
        if self.format.is_dense():
            return self
        return STensor.from_torch(self._as_torch_sparse().to_dense(), self._name)

    def to_sparse(self, fmt: Union[TensorFormat, str, List[str]] = "ds") -> "STensor":
        """Dense or sparse 2-D STensor -> "d,s" (CSR) or "o,o" (COO)."""
        fmt = parse_format(fmt)
        if fmt == self.format:
            return self
        if self.dim() != 2:
            raise NotImplementedError("to_sparse handles matrices only")
        target = str(fmt)
        if not self.format.is_dense() and target in ("d,s", "o,o"):
            # sparse -> sparse without a dense detour: the stored entries (explicit zeros
            # included) are kept, sorted by (row, column); repeated coordinates are summed
            rows, cols = self._coordinates()
            rows, cols, values = _sorted_unique_entries(rows, cols, self.values, self.shape[1])
            order = self.index.mode_order
            if target == "o,o":
                return STensor._coo(self.shape, [rows.to(torch.int32), cols.to(torch.int32)], values,
                                    self._name, order)
            pos = torch.zeros(self.shape[0] + 1, dtype=torch.int64, device=values.device)
            if rows.numel():
                pos[1:] = torch.cumsum(torch.bincount(rows, minlength=self.shape[0]), dim=0)
            return STensor._csr(self.shape, pos.to(torch.int32), cols.to(torch.int32), values, self._name, order)
        if self.format.is_dense():
            dense = self.values.reshape(self.shape)
        else:
            dense = self._as_torch_sparse().to_dense()
        if target == "d,s":
            return STensor.from_csr(dense.to_sparse_csr(), self._name)
        if target == "o,o":
            return STensor.from_coo(dense.to_sparse(), name=self._name)
        if target == "d,d":
            return STensor.from_torch(dense, self._name)
        raise NotImplementedError(f"to_sparse: unsupported target format {fmt}")

    def _coordinates(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """(rows, cols) as int64 tensors of a 2-D "d,s" or "o,o" STensor, in storage order."""
        idx = self.index.mode_indices
        if str(self.format) == "d,s":
            pos, crd = idx[1]
            if crd.is_cuda and pos.dtype == torch.int32 and crd.numel() > 0:
                from . import scorch_ops_hip
                rows = scorch_ops_hip.csr_row_indices(pos.contiguous(), int(crd.numel())).to(torch.int64)
            else:
                counts = (pos[1:] - pos[:-1]).to(torch.int64)
                rows = torch.repeat_interleave(
                    torch.arange(self.shape[0], dtype=torch.int64, device=crd.device), counts)
            return rows, crd.to(torch.int64)
        if str(self.format) == "o,o":
            return idx[0][0].to(torch.int64), idx[1][0].to(torch.int64)
        raise NotImplementedError(f"no coordinates for format {self.format}")

    def change_mode_order(self, mode_order: List[int]) -> "STensor":
        """Re-store a matrix so that its physical mode order becomes ``mode_order``
        (e.g. ``[1, 0]`` stores the transpose), in place; returns ``self``.

        Covers what the reference's 2-D fast path covers (stensor.py:785-896):
        "d,d", "d,s" and "o,o" matrices, with torch operations on whatever device
        the tensor is on.  Sparse results are sorted by (row, column) of the new
        layout and duplicate coordinates are summed.  Other tensors go through
        the reference's code generator, which is not part of this package."""
        dim = self.dim()
        if sorted(mode_order) != list(range(dim)):
            raise ValueError("mode_order must be a permutation of the modes")
        current = list(self.index.mode_order) if self.index.mode_order else list(range(dim))
        if current == list(mode_order):
            return self
        layout = str(self.format)
        if dim != 2 or layout not in ("d,d", "d,s", "o,o"):
            raise NotImplementedError(f"change_mode_order for a {dim}-D \"{layout}\" tensor")
        # mode_order[p] is the logical mode stored at physical position p
        where = {logical: physical for physical, logical in enumerate(current)}
        perm = [where[logical] for logical in mode_order]      # old physical axis of each new axis
        new_shape = tuple(self.shape[p] for p in perm)

        if layout == "d,d":
            values = self.values.reshape(self.shape).permute(*perm).contiguous().reshape(-1)
            indices = [[], []]
        else:
            if layout == "d,s":
                pos, crd = self.index.mode_indices[1]
                counts = (pos[1:] - pos[:-1]).to(torch.int64)
                rows = torch.repeat_interleave(
                    torch.arange(self.shape[0], dtype=torch.int64, device=crd.device), counts)
                coords = [rows, crd.to(torch.int64)]
            else:
                coords = [self.index.mode_indices[0][0].to(torch.int64),
                          self.index.mode_indices[1][0].to(torch.int64)]
            rows, cols, values = _sorted_unique_entries(coords[perm[0]], coords[perm[1]], self.values,
                                                        new_shape[1])
            if layout == "d,s":
                pos = torch.zeros(new_shape[0] + 1, dtype=torch.int64, device=rows.device)
                if rows.numel():
                    pos[1:] = torch.cumsum(torch.bincount(rows, minlength=new_shape[0]), dim=0)
                indices = [[], [pos.to(torch.int32), cols.to(torch.int32)]]
            else:
                indices = [[rows.to(torch.int32)], [cols.to(torch.int32)]]
        self._storage = TensorStorage(index=TensorIndex(self.format, indices, mode_order=list(mode_order)),
                                      value=values)
        self._shape = new_shape
        return self

    def to_torch(self, in_place: bool = True) -> torch.Tensor:
        """Strided torch tensor of the logical shape (reference: stensor.py:454-475);
        no copy for a dense STensor in default mode order."""
        if self.format.is_dense():
            out = self.values
        else:
            out = self._as_torch_sparse().to_dense()
        if out.dtype != self.dtype:
            out = out.to(self.dtype)
        out = out.reshape(self.shape)
        order = self.index.mode_order
        if order and list(order) != list(range(self.dim())):
            inverse = [0] * len(order)
            for pos, mode in enumerate(order):
                inverse[mode] = pos
            out = out.permute(*inverse)
        return out
