"""``@tunable`` kernels and the pruned grid search over their tile configs.

Interface and search order follow tritonix/autotune.py of the reference:
``tunable`` (:217-227), ``TunableKernel`` (:21-73) and ``_tune_grid``
(:75-140).  The outer loop walks the memory parameters (block sizes and
``num_stages``) centre-out through a ``MonotonicCascadeTrie``; the inner loop
walks the remaining parameters in declaration order; a
``CoordinateUnimodalFunction`` skips configs that cannot hold the minimum; a
launcher that raises ``ValueError`` vetoes one config; one that raises
``OutOfResources`` prunes every config at least as large in all memory
parameters.

Two things differ from the reference on purpose.  The trie's dimension order
is the declaration order of ``space`` (the reference iterates a ``set``,
tritonix/autotune.py:39, so its order changes from process to process).  And
``OutOfResources`` is raised by the HIP launcher from host arithmetic -- the
tile's LDS bytes against the 160 KiB a CU has -- before anything is launched,
where Triton raised it from a failed compile.
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Set

from tritonix_amd.testing import OutOfResources, do_bench
from tritonix_amd.utils.pruners import CoordinateMonotonicFunction, MonotonicCascadeTrie
from tritonix_amd.utils.spaces import Choice, ConfigParam, PowerOfTwo, Range, SpaceConfig

__all__ = ["tunable", "TunableKernel", "PowerOfTwo", "Range", "Choice", "SpaceConfig", "OutOfResources"]


@dataclass
class TunableKernel:
    kernel: Any
    keys: List[str]
    space: Dict[str, ConfigParam]
    memory_params: Set[str]

    def __post_init__(self):
        if isinstance(self.kernel, TunableKernel):
            self.kernel = self.kernel.kernel

    # anything that is not a tuner attribute is the wrapped kernel's
    def __getattr__(self, name):
        if name in ("kernel", "__setstate__", "__getstate__"):
            raise AttributeError(name)
        return getattr(self.kernel, name)

    def __getitem__(self, grid):
        return self.kernel[grid]

    # ------------------------------------------------------------------
    def _build_trie(self):
        names = [p for p in self.space if p in self.memory_params]
        values = [sorted(self.space[p].values()) for p in names]
        trie = MonotonicCascadeTrie(SpaceConfig({n: Choice(v) for n, v in zip(names, values)}))
        return trie, names, values

    def configs(self, filter_fn: Optional[Callable[[dict], bool]] = None) -> List[dict]:
        """Every config of the space, first parameter varying slowest."""
        names = list(self.space)
        out = [dict(zip(names, combo)) for combo in itertools.product(*(self.space[n].values() for n in names))]
        if filter_fn is not None:
            out = [c for c in out if filter_fn(c)]
        return out

    def tune(self, launcher: Callable[[dict], Any], method: str = "grid", max_configs: Optional[int] = None,
             max_evals: int = 100, filter_fn: Optional[Callable[[dict], bool]] = None, warmup: float = 25,
             rep: float = 100, verbose: bool = False, bench_fn: Optional[Callable] = None):
        """Best config dict for ``launcher(cfg)``, or ``None`` if nothing ran.

        ``bench_fn(fn, warmup=, rep=)`` replaces the HIP-event timer (tests
        pass a deterministic table).
        """
        timer = bench_fn or do_bench
        if method == "grid":
            return self._tune_grid(launcher, max_configs, filter_fn, warmup, rep, verbose, timer)
        return self._tune_bayesian(launcher, max_evals, filter_fn, warmup, rep, verbose, timer)

    # ------------------------------------------------------------------
    def _tune_grid(self, launcher, max_configs, filter_fn, warmup, rep, verbose, timer=do_bench):
        trie, mem_names, mem_values = self._build_trie()

        names = list(self.space)
        values = [sorted(self.space[n].values()) for n in names]
        index_of = [{v: i for i, v in enumerate(vals)} for vals in values]
        perf = CoordinateMonotonicFunction(SpaceConfig({n: Choice(v) for n, v in zip(names, values)}))

        mem_set = set(mem_names)
        free_names = [n for n in names if n not in mem_set]
        free_values = [values[names.index(n)] for n in free_names]

        best_ms, best_cfg, evaluated = float("inf"), None, 0
        capped = (lambda: max_configs is not None and evaluated >= max_configs)

        for mem_idx in trie.generate_all_unpruned_midpoint():
            if capped():
                break
            mem_cfg = {n: mem_values[d][mem_idx[d]] for d, n in enumerate(mem_names)}
            for combo in itertools.product(*free_values):
                if capped():
                    break
                cfg = {**mem_cfg, **dict(zip(free_names, combo))}
                if filter_fn is not None and not filter_fn(cfg):
                    continue
                pos = tuple(index_of[d][cfg[n]] for d, n in enumerate(names))
                if perf.is_pruned(pos):
                    continue
                try:
                    ms = timer(lambda: launcher(cfg), warmup=warmup, rep=rep)
                except ValueError as exc:
                    if verbose:
                        print(f"  SKIP      {cfg}  ({exc})", flush=True)
                    continue
                except OutOfResources:
                    trie.prune(mem_idx)
                    if verbose:
                        print(f"  OOM       {cfg}", flush=True)
                    break
                perf.record(pos, ms)
                evaluated += 1
                improved = ms < best_ms
                if improved:
                    best_ms, best_cfg = ms, cfg
                if verbose:
                    print(f"  {ms:8.3f}ms  {cfg}{' *' if improved else ''}", flush=True)
        return best_cfg

    def _tune_bayesian(self, launcher, max_evals, filter_fn, warmup, rep, verbose, timer=do_bench, oom_penalty=1e6):
        """Ax-driven search (tritonix/autotune.py:142-214); needs the optional ``ax-platform`` package."""
        try:
            from ax.service.ax_client import AxClient
            from ax.service.utils.instantiation import ObjectiveProperties
        except ImportError as exc:  # same failure mode as the reference when Ax is absent
            raise ImportError("method='bayesian' needs the optional 'ax-platform' package; use method='grid'") from exc

        trie, mem_names, mem_values = self._build_trie()
        ax_params = [{"name": n, "type": "choice", "values": p.values(), "sort_values": True,
                      "is_ordered": isinstance(p, (PowerOfTwo, Range))}
                     for n, p in self.space.items() if len(p.values()) > 1]
        client = AxClient(verbose_logging=False)
        client.create_experiment(name="kernel_tune", parameters=ax_params,
                                 objectives={"latency_ms": ObjectiveProperties(minimize=True)})
        fixed = {n: p.values()[0] for n, p in self.space.items() if len(p.values()) == 1}

        def mem_pos(cfg):
            return tuple(mem_values[d].index(cfg[n]) for d, n in enumerate(mem_names))

        for i in range(max_evals):
            params, trial = client.get_next_trial()
            cfg = {**fixed, **params}
            dead = bool(mem_names) and trie.is_pruned(mem_pos(cfg))
            dead = dead or (filter_fn is not None and not filter_fn(cfg))
            if dead:
                client.complete_trial(trial_index=trial, raw_data={"latency_ms": oom_penalty})
                continue
            try:
                ms = timer(lambda: launcher(cfg), warmup=warmup, rep=rep)
                client.complete_trial(trial_index=trial, raw_data={"latency_ms": ms})
                if verbose:
                    print(f"  [{i + 1}/{max_evals}] {ms:.3f}ms - {cfg}")
            except OutOfResources:
                if mem_names:
                    trie.prune(mem_pos(cfg))
                client.complete_trial(trial_index=trial, raw_data={"latency_ms": oom_penalty})
        best, _ = client.get_best_parameters()
        return {**fixed, **best}


def tunable(keys, space, memory_params=None):
    """Decorator: wrap a kernel in a ``TunableKernel``; ``num_stages`` always counts as a memory parameter."""
    mem = set(memory_params or set()) | {"num_stages"}

    def wrap(kernel):
        t = TunableKernel(kernel=kernel, keys=keys, space=space, memory_params=mem)
        t.kernel.specialize_keys = keys
        return t

    return wrap
