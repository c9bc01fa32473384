"""Level formats of a stored tensor, with the reference's spelling.

A tensor format is one level type per mode: dense "d", compressed "s"
(CSR's second level), coordinate "o".  ``str(TensorFormat)`` is the
comma-joined level letters ("d,s", "d,d", "o,o"): the prebuilt-kernel registry
matches on exactly these strings (reference: src/scorch/format.py:7-27,
130-133; src/scorch/utils.py:333-357 for the accepted aliases).
"""
from __future__ import annotations

from enum import Enum
from typing import Iterable, List, Union


class LevelType(Enum):
    DENSE = "d"
    COMPRESSED = "s"
    SINGLETON = "singleton"
    COORDINATE = "o"


_ALIASES = {
    "dense": LevelType.DENSE, "d": LevelType.DENSE,
    "compressed": LevelType.COMPRESSED, "sparse": LevelType.COMPRESSED,
    "c": LevelType.COMPRESSED, "s": LevelType.COMPRESSED,
    "singleton": LevelType.SINGLETON, "single": LevelType.SINGLETON,
    "coordinate": LevelType.COORDINATE, "coord": LevelType.COORDINATE, "o": LevelType.COORDINATE,
}


def level_type_of(name: Union[str, LevelType]) -> LevelType:
    if isinstance(name, LevelType):
        return name
    try:
        return _ALIASES[name]
    except KeyError:
        raise ValueError(f"Invalid format string: {name}") from None


class LevelFormat:
    """The storage of one mode."""

    def __init__(self, mode: Union[str, LevelType]):
        self._mode = level_type_of(mode)

    def get_level_type(self) -> LevelType:
        return self._mode

    def __str__(self) -> str:
        return str(self._mode.value)

    __repr__ = __str__

    def __eq__(self, other) -> bool:
        return isinstance(other, LevelFormat) and self._mode == other._mode

    def __hash__(self) -> int:
        return hash(self._mode)


class TensorFormat:
    """One LevelFormat per mode."""

    def __init__(self, level_formats: Union[None, str, LevelFormat, Iterable] = None):
        if level_formats is None:
            levels: List[LevelFormat] = []
        elif isinstance(level_formats, LevelFormat):
            levels = [level_formats]
        else:
            if isinstance(level_formats, str):
                level_formats = list(level_formats)
            levels = [lf if isinstance(lf, LevelFormat) else LevelFormat(lf) for lf in level_formats]
        self._level_formats = levels

    def get_level_formats(self) -> List[LevelFormat]:
        return self._level_formats

    def get_level_types(self) -> List[LevelType]:
        return [lf.get_level_type() for lf in self._level_formats]

    def get_order(self) -> int:
        return len(self._level_formats)

    def is_dense(self) -> bool:
        return all(t == LevelType.DENSE for t in self.get_level_types())

    def __str__(self) -> str:
        return ",".join(str(lf) for lf in self._level_formats)

    __repr__ = __str__

    def __eq__(self, other) -> bool:
        return isinstance(other, TensorFormat) and self._level_formats == other._level_formats

    def __ne__(self, other) -> bool:
        return not self.__eq__(other)

    def __hash__(self) -> int:
        return hash(str(self))


def parse_format(fmt: Union[TensorFormat, str, Iterable[str]]) -> TensorFormat:
    """"ds", ["dense", "compressed"] or a TensorFormat -> TensorFormat.
    Only dense / compressed / coordinate levels may be requested this way
    (reference: src/scorch/utils.py:333-357)."""
    if isinstance(fmt, TensorFormat):
        return fmt
    names = list(fmt)
    levels = []
    for name in names:
        kind = _ALIASES.get(name)
        if kind is None or kind == LevelType.SINGLETON:
            raise ValueError(f"Invalid format string: {name}")
        levels.append(LevelFormat(kind))
    return TensorFormat(levels)
