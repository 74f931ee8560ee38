"""``@tunable`` kernels and the pruned search over their tile configs.

What a caller sees follows the reference's tuner (tritonix/autotune.py:
``tunable`` :217-227, ``TunableKernel`` :21-73, the grid search :75-140, the
Ax search :142-214): a kernel wrapped by ``@tunable(keys, space,
memory_params)`` keeps its launch syntax and gains ``configs()`` and
``tune(launcher, ...)``.  The grid search visits the memory parameters (block
sizes, ``num_stages``) from the centre of their ranges outwards and, under
each of those points, the remaining parameters in declaration order.  Three
things thin the walk: a launcher that raises ``OutOfResources`` rules out
every point at least as large in all memory parameters (a
``MonotonicCascadeTrie`` holds those verdicts), one that raises ``ValueError``
rules out just that config, and a ``CoordinateUnimodalFunction`` rules out
configs that lie beyond a point already seen to be worse along one axis.

Deliberate differences.  The memory axes keep the declaration order of
``space`` (the reference iterates a ``set``, tritonix/autotune.py:39, so its
visit order changes from process to process).  ``OutOfResources`` comes from
host arithmetic in the HIP launcher -- the tile's LDS bytes against the 160
KiB of a CU -- before anything is launched, where Triton raised it from a
failed compile.  ``tune`` accepts ``bench_fn`` to replace the HIP-event timer.
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass
from typing import Any, Callable, Dict, Iterator, List, Optional, Sequence, Set, Tuple

from tritonix_amd.testing import OutOfResources, do_bench
from tritonix_amd.utils.pruners import CoordinateMonotonicFunction, MonotonicCascadeTrie
from tritonix_amd.utils.spaces import Choice, ConfigParam, PowerOfTwo, Range, SpaceConfig

__all__ = ["tunable", "TunableKernel", "PowerOfTwo", "Range", "Choice", "SpaceConfig", "OutOfResources"]


class _Axes:
    """A subset of a space's parameters, in declaration order, with their values sorted ascending."""

    def __init__(self, space: Dict[str, ConfigParam], keep: Callable[[str], bool]):
        self.names: List[str] = [name for name in space if keep(name)]
        self.values: List[List[Any]] = [sorted(space[name].values()) for name in self.names]

    def as_space(self) -> SpaceConfig:
        return SpaceConfig({name: Choice(vals) for name, vals in zip(self.names, self.values)})

    def at(self, index: Sequence[int]) -> Dict[str, Any]:
        return {name: vals[i] for name, vals, i in zip(self.names, self.values, index)}

    def locate(self, cfg: Dict[str, Any]) -> Tuple[int, ...]:
        return tuple(vals.index(cfg[name]) for name, vals in zip(self.names, self.values))

    def combinations(self) -> Iterator[Dict[str, Any]]:
        for combo in itertools.product(*self.values):
            yield dict(zip(self.names, combo))


class _GridSearch:
    """State of one pruned walk over a space: verdicts so far, the best config, how many were timed."""

    def __init__(self, space: Dict[str, ConfigParam], memory_params: Set[str], limit: Optional[int], accept, echo):
        self.everything = _Axes(space, lambda name: True)
        self.memory = _Axes(space, lambda name: name in memory_params)
        self.rest = _Axes(space, lambda name: name not in memory_params)
        self.too_big = MonotonicCascadeTrie(self.memory.as_space())
        self.shape_of_f = CoordinateMonotonicFunction(self.everything.as_space())
        self.limit, self.accept, self.echo = limit, accept, echo
        self.timed = 0
        self.best_ms, self.best = float("inf"), None

    def _full(self) -> bool:
        return self.limit is not None and self.timed >= self.limit

    def run(self, launcher, clock, budget) -> Optional[dict]:
        for corner in self.too_big.generate_all_unpruned_midpoint():
            if self._full():
                break
            self._under(corner, launcher, clock, budget)
        return self.best

    def _under(self, corner, launcher, clock, budget) -> None:
        """All configs that share one point of the memory axes; stops at the first one that does not fit."""
        fixed = self.memory.at(corner)
        for tail in self.rest.combinations():
            if self._full():
                return
            cfg = {**fixed, **tail}
            if self.accept is not None and not self.accept(cfg):
                continue
            where = self.everything.locate(cfg)
            if self.shape_of_f.is_pruned(where):
                continue
            try:
                ms = clock(lambda: launcher(cfg), **budget)
            except ValueError as why:
                self.echo(f"  SKIP      {cfg}  ({why})")
                continue
            except OutOfResources:
                self.too_big.prune(corner)
                self.echo(f"  OOM       {cfg}")
                return
            self.shape_of_f.record(where, ms)
            self.timed += 1
            better = ms < self.best_ms
            if better:
                self.best_ms, self.best = ms, cfg
            self.echo(f"  {ms:8.3f}ms  {cfg}{' *' if better else ''}")


@dataclass
class TunableKernel:
    kernel: Any
    keys: List[str]
    space: Dict[str, ConfigParam]
    memory_params: Set[str]

    def __post_init__(self):
        inner = self.kernel
        if isinstance(inner, TunableKernel):          # decorating twice wraps the same kernel once
            self.kernel = inner.kernel

    def __getattr__(self, name):
        # only reached for names the dataclass does not hold: hand them to the wrapped kernel
        if name in ("kernel", "__setstate__", "__getstate__"):
            raise AttributeError(name)
        return getattr(self.kernel, name)

    def __getitem__(self, grid):
        return self.kernel[grid]

    def _build_trie(self):
        """(trie over the memory parameters, their names in declaration order, their sorted values)."""
        axes = _Axes(self.space, lambda name: name in self.memory_params)
        return MonotonicCascadeTrie(axes.as_space()), axes.names, axes.values

    def configs(self, filter_fn: Optional[Callable[[dict], bool]] = None) -> List[dict]:
        """The whole space as config dicts, last parameter varying fastest, values in the order the domains list them."""
        names = list(self.space)
        domains = [self.space[name].values() for name in names]
        every = (dict(zip(names, point)) for point in itertools.product(*domains))
        return [cfg for cfg in every if filter_fn is None or filter_fn(cfg)]

    def tune(self, launcher: Callable[[dict], Any], method: str = "grid", max_configs: Optional[int] = None,
             max_evals: int = 100, filter_fn: Optional[Callable[[dict], bool]] = None, warmup: float = 25,
             rep: float = 100, verbose: bool = False, bench_fn: Optional[Callable] = None):
        """The fastest config found for ``launcher(cfg)``, or ``None`` when no config could be timed.

        ``method="grid"`` is the pruned walk (``max_configs`` caps how many configs are timed);
        anything else is the Ax search (``max_evals`` trials).
        """
        clock = bench_fn if bench_fn is not None else do_bench
        if method == "grid":
            return self._tune_grid(launcher, max_configs, filter_fn, warmup, rep, verbose, clock)
        return self._tune_bayesian(launcher, max_evals, filter_fn, warmup, rep, verbose, clock)

    def _tune_grid(self, launcher, max_configs, filter_fn, warmup, rep, verbose, timer=do_bench):
        echo = (lambda line: print(line, flush=True)) if verbose else (lambda line: None)
        search = _GridSearch(self.space, self.memory_params, max_configs, filter_fn, echo)
        return search.run(launcher, timer, {"warmup": warmup, "rep": rep})

    def _tune_bayesian(self, launcher, max_evals, filter_fn, warmup, rep, verbose, timer=do_bench, oom_penalty=1e6):
        """Model-based search through Ax; the optional ``ax-platform`` package must be installed."""
        try:
            from ax.service.ax_client import AxClient
            from ax.service.utils.instantiation import ObjectiveProperties
        except ImportError as missing:
            raise ImportError("method='bayesian' needs the optional 'ax-platform' package; use method='grid'") from missing

        memory = _Axes(self.space, lambda name: name in self.memory_params)
        too_big = MonotonicCascadeTrie(memory.as_space()) if memory.names else None
        constant = {name: dom.values()[0] for name, dom in self.space.items() if len(dom.values()) == 1}
        searched = [{"name": name, "type": "choice", "values": dom.values(), "sort_values": True,
                     "is_ordered": isinstance(dom, (PowerOfTwo, Range))}
                    for name, dom in self.space.items() if name not in constant]
        ax = AxClient(verbose_logging=False)
        ax.create_experiment(name="kernel_tune", parameters=searched,
                             objectives={"latency_ms": ObjectiveProperties(minimize=True)})

        def report(trial, ms):
            ax.complete_trial(trial_index=trial, raw_data={"latency_ms": ms})

        for attempt in range(1, max_evals + 1):
            proposal, trial = ax.get_next_trial()
            cfg = {**constant, **proposal}
            known_bad = too_big is not None and too_big.is_pruned(memory.locate(cfg))
            if known_bad or (filter_fn is not None and not filter_fn(cfg)):
                report(trial, oom_penalty)          # steer the model away without launching anything
                continue
            try:
                ms = timer(lambda: launcher(cfg), warmup=warmup, rep=rep)
            except OutOfResources:
                if too_big is not None:
                    too_big.prune(memory.locate(cfg))
                report(trial, oom_penalty)
                continue
            report(trial, ms)
            if verbose:
                print(f"  [{attempt}/{max_evals}] {ms:.3f}ms - {cfg}")
        winner, _ = ax.get_best_parameters()
        return {**constant, **winner}


def tunable(keys, space, memory_params=None):
    """Decorator factory: ``@tunable(keys=[...], space={...}, memory_params={...})``.

    ``keys`` name the launch arguments a tuned config is specific to (they are also set as the kernel's
    ``specialize_keys``); ``num_stages`` is always treated as a memory parameter.
    """
    memory = set(memory_params) if memory_params else set()
    memory.add("num_stages")

    def decorate(kernel):
        wrapped = TunableKernel(kernel=kernel, keys=keys, space=space, memory_params=memory)
        wrapped.kernel.specialize_keys = keys
        return wrapped

    return decorate
