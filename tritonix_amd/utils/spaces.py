"""Parameter domains of a tuning space.

Behaviour follows tritonix/utils/spaces.py of the reference:
``Choice`` (:7-23) is an explicit list, ``Range`` (:26-40) is an integer
progression whose upper bound is *inclusive*, ``PowerOfTwo`` (:43-62) doubles
from ``lo`` while the value stays ``<= hi`` (``lo`` itself need not be a power
of two), and ``SpaceConfig`` (:68-86) is an ordered mapping of such domains
with a ``shape``, index-tuple lookup and a product ``len``.  The docs of the
reference call the last one ``ConfigSpace``; both names are exported.
"""
from __future__ import annotations

import math
from typing import Any, Dict, Iterable, List, Tuple, Union

__all__ = ["Choice", "Range", "PowerOfTwo", "ConfigParam", "SpaceConfig", "ConfigSpace"]


class _Domain:
    """Shared list-like behaviour: every domain is defined by ``values()``."""

    def values(self) -> List[Any]:  # pragma: no cover - overridden
        raise NotImplementedError

    def __len__(self) -> int:
        return len(self.values())

    def __getitem__(self, idx):
        return self.values()[idx]

    def __iter__(self):
        return iter(self.values())

    def __eq__(self, other):
        return type(other) is type(self) and self._key() == other._key()

    def __hash__(self):
        return hash((type(self).__name__, self._key()))


class Choice(_Domain):
    """An explicit list of allowed values, kept in the order given."""

    def __init__(self, options: Iterable[Any]):
        self.options = list(options)

    def values(self) -> List[Any]:
        return list(self.options)

    def _key(self):
        return tuple(self.options)

    def __repr__(self):
        return f"Choice(options={self.options!r})"


class Range(_Domain):
    """Integers ``lo, lo+step, ...`` up to and including ``hi``."""

    def __init__(self, lo: int, hi: int, step: int = 1):
        self.lo, self.hi, self.step = lo, hi, step

    def values(self) -> List[int]:
        return list(range(self.lo, self.hi + 1, self.step))

    def __getitem__(self, idx):
        # arithmetic, not list lookup: the reference does not bounds-check here
        if isinstance(idx, slice):
            return self.values()[idx]
        return self.lo + idx * self.step

    def _key(self):
        return (self.lo, self.hi, self.step)

    def __repr__(self):
        return f"Range(lo={self.lo}, hi={self.hi}, step={self.step})"


class PowerOfTwo(_Domain):
    """``lo, 2*lo, 4*lo, ...`` while the value is ``<= hi``."""

    def __init__(self, lo: int, hi: int):
        self.lo, self.hi = lo, hi

    def values(self) -> List[int]:
        out, v = [], self.lo
        if v <= 0:
            return out
        while v <= self.hi:
            out.append(v)
            v *= 2
        return out

    def _key(self):
        return (self.lo, self.hi)

    def __repr__(self):
        return f"PowerOfTwo(lo={self.lo}, hi={self.hi})"


ConfigParam = Union[PowerOfTwo, Range, Choice]


class SpaceConfig:
    """Ordered ``name -> domain`` mapping; every domain must be non-empty."""

    def __init__(self, params: Dict[str, ConfigParam]):
        self.params = dict(params)
        for name, dom in self.params.items():
            if len(dom) == 0:
                raise ValueError(f"Param '{name}' has no values.")

    @property
    def shape(self) -> Tuple[int, ...]:
        return tuple(len(dom) for dom in self.params.values())

    @property
    def names(self) -> List[str]:
        return list(self.params)

    def __getitem__(self, idx_tuple):
        if len(idx_tuple) != len(self.params):
            raise AssertionError("index tuple length must equal the number of parameters")
        return [dom[i] for dom, i in zip(self.params.values(), idx_tuple)]

    def __len__(self) -> int:
        return math.prod(len(dom) for dom in self.params.values())

    def __repr__(self):
        return f"SpaceConfig(params={self.params!r})"


ConfigSpace = SpaceConfig
