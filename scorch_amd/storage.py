"""Index and value storage of an STensor (reference: src/scorch/storage.py).

``TensorIndex.mode_indices`` is a list, one entry per mode, of lists of index
tensors: ``[[], []]`` for a dense matrix, ``[[], [pos, crd]]`` for CSR,
``[[row], [col]]`` for coordinate format.  Every index tensor is converted to
int32 on construction (reference: storage.py:46-51): the kernels read int32.
"""
from __future__ import annotations

from typing import List, Optional, Tuple, Union

import torch

from .format import LevelType, TensorFormat, parse_format


class TensorIndex:
    def __init__(self, tensor_format: Optional[Union[TensorFormat, str, List[str]]] = None,
                 mode_indices: Optional[List[List[torch.Tensor]]] = None,
                 mode_order: Optional[List[int]] = None):
        self.format = parse_format(tensor_format) if tensor_format else None
        self.mode_indices = mode_indices
        if self.mode_indices:
            for level in self.mode_indices:
                for k, idx in enumerate(level):
                    if idx.dtype != torch.int32:
                        level[k] = idx.to(torch.int32)
        self.mode_order = list(mode_order) if mode_order else list(range(self.get_order()))

    def __repr__(self) -> str:
        return f"TensorIndex({self.format})"

    def __eq__(self, other) -> bool:
        if not isinstance(other, TensorIndex) or self.format != other.format:
            return False
        mine, theirs = self.mode_indices or [], other.mode_indices or []
        if len(mine) != len(theirs):
            return False
        for la, lb in zip(mine, theirs):
            if len(la) != len(lb) or any(not torch.equal(a, b) for a, b in zip(la, lb)):
                return False
        return True

    def __ne__(self, other) -> bool:
        return not self.__eq__(other)

    def copy(self) -> "TensorIndex":
        indices = None
        if self.mode_indices is not None:
            indices = [[t.clone().detach() for t in level] for level in self.mode_indices]
        return TensorIndex(self.format, indices, mode_order=list(self.mode_order))

    def to(self, device) -> "TensorIndex":
        indices = None
        if self.mode_indices is not None:
            indices = [[t.to(device) for t in level] for level in self.mode_indices]
        return TensorIndex(self.format, indices, mode_order=list(self.mode_order))

    def get_mode_indices(self) -> List[List[torch.Tensor]]:
        assert self.mode_indices is not None, "mode_indices is None"
        return self.mode_indices

    def get_mode_index(self, mode: int) -> List[torch.Tensor]:
        return self.get_mode_indices()[mode]

    def get_format(self) -> TensorFormat:
        assert self.format is not None, "format is None"
        return self.format

    def get_order(self) -> int:
        return self.get_format().get_order()

    def get_mode_order(self) -> List[int]:
        return self.mode_order

    def get_level_types(self) -> List[LevelType]:
        return self.get_format().get_level_types()

    def get_level_type(self, mode: int) -> LevelType:
        return self.get_level_types()[mode]


class TensorStorage:
    def __init__(self, index: Optional[TensorIndex] = None, value: Optional[torch.Tensor] = None,
                 shape: Optional[Tuple[int, ...]] = None):
        self._index = index
        self._value = value
        self._shape = shape

    def __repr__(self) -> str:
        return "TensorStorage({})"

    def copy(self) -> "TensorStorage":
        return TensorStorage(index=self._index.copy() if self._index is not None else None,
                             value=self._value.clone() if self._value is not None else None,
                             shape=self._shape)

    def to(self, device) -> "TensorStorage":
        return TensorStorage(index=self._index.to(device) if self._index is not None else None,
                             value=self._value.to(device) if self._value is not None else None,
                             shape=self._shape)

    @property
    def has_index(self) -> bool:
        return self._index is not None

    @property
    def value(self) -> torch.Tensor:
        assert self._value is not None, "value is None"
        return self._value

    @property
    def index(self) -> TensorIndex:
        assert self._index is not None, "index is None"
        return self._index
