"""Search-space pruners used by the tile-config tuner.

``MonotonicCascadeTrie`` keeps the antichain of minimal failing index tuples of
a space in which failure is monotone (a config that needs too much LDS still
does after any coordinate grows) and enumerates what is left; behaviour
follows tritonix/utils/pruners.py:15-169 of the reference, pinned by the
reference's tests/test_trie.py.  ``CoordinateUnimodalFunction`` narrows, per
one-dimensional slice, the index window that can still hold the minimum of a
coordinate-wise unimodal function; behaviour follows
tritonix/utils/pruners.py:172-225.  The reference's tuner imports that class
under the name ``CoordinateMonotonicFunction`` (tritonix/autotune.py:8-11), so
both names are bound to it here.
"""
from __future__ import annotations

import random
from typing import Callable, Dict, Iterator, List, Optional, Sequence, Tuple

from tritonix_amd.utils.spaces import SpaceConfig

__all__ = ["MonotonicCascadeTrie", "CoordinateUnimodalFunction", "CoordinateMonotonicFunction"]


def _dominates_config(failure: Sequence[int], candidate: Sequence[int]) -> bool:
    """candidate is at least failure in every coordinate"""
    return all(c >= f for c, f in zip(candidate, failure))


def _dominates_dim(failure: int, candidate: int, rank: int = 0) -> bool:
    return candidate >= failure


class _Node:
    __slots__ = ("kids", "terminal")

    def __init__(self):
        self.kids: Dict[int, "_Node"] = {}
        self.terminal = False


def _centre_out(n: int) -> Iterator[int]:
    """n//2, then alternately one step below and one step above, until 0..n-1 is used up."""
    mid = n // 2
    yield mid
    below, above = mid - 1, mid + 1
    while below >= 0 or above < n:
        if below >= 0:
            yield below
            below -= 1
        if above < n:
            yield above
            above += 1


class MonotonicCascadeTrie:
    """Prefix tree over the minimal failures of a monotone search space."""

    def __init__(self, space: SpaceConfig, config_comparison_func: Callable = _dominates_config,
                 dimension_comparison_func: Callable = _dominates_dim):
        self.shape = space.shape
        self.dimensions = len(self.shape)
        self._minimal_failures: List[Tuple[int, ...]] = []
        self._root = _Node()
        self._config_compare = config_comparison_func
        self._dim_compare = dimension_comparison_func

    # -- queries ---------------------------------------------------------
    def is_pruned(self, config_idx) -> bool:
        """True when some recorded failure is <= config_idx in every coordinate."""
        if len(config_idx) != self.dimensions:
            raise ValueError(f"is_pruned expects a full-length config of length {self.dimensions}")
        return self._covered(tuple(config_idx), 0, self._root)

    def _covered(self, cfg: Tuple[int, ...], depth: int, node: _Node) -> bool:
        if node.terminal:
            return True
        if depth == len(cfg):
            return False
        here = cfg[depth]
        for fail_idx, child in node.kids.items():
            if self._dim_compare(fail_idx, here, depth) and self._covered(cfg, depth + 1, child):
                return True
        return False

    def _is_prefix_doomed(self, prefix) -> bool:
        """A prefix is dead when even its all-zero completion is pruned."""
        prefix = tuple(prefix)
        if not prefix:
            return False
        return self.is_pruned(prefix + (0,) * (self.dimensions - len(prefix)))

    # -- updates ---------------------------------------------------------
    def prune(self, failed_config) -> None:
        """Record a failure; failures it makes redundant are dropped."""
        if self.is_pruned(failed_config):
            return
        kept = [f for f in self._minimal_failures if not self._config_compare(failed_config, f)]
        kept.append(failed_config)
        self._minimal_failures = kept
        self._root = _Node()
        for f in kept:
            node = self._root
            for idx in f:
                node = node.kids.setdefault(idx, _Node())
            node.terminal = True

    # -- enumeration -----------------------------------------------------
    def _first_survivor(self, prefix: Tuple[int, ...], order: Callable[[int], Sequence[int]]) -> Optional[Tuple[int, ...]]:
        if self._is_prefix_doomed(prefix):
            return None
        if len(prefix) == self.dimensions:
            return prefix
        for idx in order(self.shape[len(prefix)]):
            found = self._first_survivor(prefix + (idx,), order)
            if found is not None:
                return found
        return None

    def get_random_unpruned(self) -> Optional[Tuple[int, ...]]:
        def shuffled(n):
            idx = list(range(n))
            random.shuffle(idx)
            return idx

        return self._first_survivor((), shuffled)

    def get_mid_point_unpruned(self) -> Optional[Tuple[int, ...]]:
        return self._first_survivor((), lambda n: list(_centre_out(n)))

    def _walk(self, prefix: Tuple[int, ...], order: Callable[[int], Sequence[int]]) -> Iterator[Tuple[int, ...]]:
        # lazy on purpose: a prune() issued by the consumer between two
        # yields changes what is produced afterwards
        if self._is_prefix_doomed(prefix):
            return
        if len(prefix) == self.dimensions:
            yield prefix
            return
        for idx in order(self.shape[len(prefix)]):
            yield from self._walk(prefix + (idx,), order)

    def generate_all_unpruned(self) -> Iterator[Tuple[int, ...]]:
        """Surviving index tuples in lexicographic order."""
        yield from self._walk((), range)

    def generate_all_unpruned_midpoint(self) -> Iterator[Tuple[int, ...]]:
        """Surviving index tuples, every dimension visited centre-out."""
        yield from self._walk((), _centre_out)


class CoordinateUnimodalFunction:
    """Coordinate-wise unimodality pruner.

    Fix all coordinates but one: along the free one the function is assumed to
    have a single minimum.  After two or more observations in such a slice,
    the first observation right of the best one that is strictly worse caps
    the window from above, the first one left of it that is strictly worse
    caps it from below.  A config outside the window of any of its slices is
    pruned.  Windows are recomputed from all observations at every record.
    """

    def __init__(self, space: SpaceConfig):
        self.dim_sizes = list(space.shape)
        self.n_dims = len(self.dim_sizes)
        self._obs: List[Dict[tuple, Dict[int, float]]] = [dict() for _ in range(self.n_dims)]
        self._ranges: List[Dict[tuple, Tuple[int, int]]] = [dict() for _ in range(self.n_dims)]

    @staticmethod
    def _slice_key(idx: Tuple[int, ...], d: int) -> tuple:
        return idx[:d] + idx[d + 1:]

    def record(self, config_idx, value: float) -> None:
        config_idx = tuple(config_idx)
        for d in range(self.n_dims):
            key = self._slice_key(config_idx, d)
            seen = self._obs[d].setdefault(key, {})
            seen[config_idx[d]] = value
            if len(seen) < 2:
                continue
            best = min(seen, key=seen.__getitem__)
            floor = seen[best]
            lo, hi = 0, self.dim_sizes[d] - 1
            for i in sorted(seen):
                if i > best and seen[i] > floor:
                    hi = i - 1
                    break
            for i in sorted(seen, reverse=True):
                if i < best and seen[i] > floor:
                    lo = i + 1
                    break
            if lo > 0 or hi < self.dim_sizes[d] - 1:
                self._ranges[d][key] = (lo, hi)

    def is_pruned(self, config_idx) -> bool:
        config_idx = tuple(config_idx)
        for d in range(self.n_dims):
            window = self._ranges[d].get(self._slice_key(config_idx, d))
            if window is not None and not (window[0] <= config_idx[d] <= window[1]):
                return True
        return False


CoordinateMonotonicFunction = CoordinateUnimodalFunction
