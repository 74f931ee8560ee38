"""Per-shape backend dispatch: time every registered implementation once, keep the fastest.

API and behaviour follow tritonix/dispatcher.py of the reference:
``_tuning_key`` (:18-30), ``_disk_key`` (:33-35), ``DynamicDispatcher``
(:38-145) and ``dynamic_dispatch`` (:148-175).  The on-disk record keeps the
reference's JSON schema ``{"op", "key", "winner", "timings"}`` and file name,
but lives under ``$TRITONIX_CACHE_DIR`` (default ``~/.cache/tritonix_amd``)
instead of Triton's cache directory, and the timer is the HIP-event
``do_bench`` of this package (or any callable passed as ``bench_fn``).
"""
from __future__ import annotations

import hashlib
import inspect
import json
import logging
import os
import tempfile
from contextlib import contextmanager
from typing import Callable, Dict, List, Optional

log = logging.getLogger(__name__)

__all__ = ["DynamicDispatcher", "dynamic_dispatch", "cache_dir"]


def cache_dir() -> str:
    return os.environ.get("TRITONIX_CACHE_DIR") or os.path.join(os.path.expanduser("~"), ".cache", "tritonix_amd")


def _is_tensor(v) -> bool:
    return hasattr(v, "shape") and hasattr(v, "dtype") and hasattr(v, "stride")


def _describe(v) -> list:
    return list(v.shape) + [str(v.dtype)]


def _tuning_key(key_names: List[str], args: tuple, kwargs: dict, arg_names: List[str]) -> tuple:
    """Shapes and dtypes of the keyed tensors, values of keyed scalars, then every other tensor argument."""
    bound = dict(zip(arg_names, args))
    bound.update(kwargs)
    parts: list = []
    for name in key_names:
        if name in bound:
            v = bound[name]
            parts.extend(_describe(v) if _is_tensor(v) else [v])
    keyed = set(key_names)
    for name, v in bound.items():
        if name not in keyed and _is_tensor(v):
            parts.extend(_describe(v))
    return tuple(parts)


def _disk_key(op_name: str, backends: List[str], tuning_key: tuple) -> str:
    text = "-".join([op_name, str(sorted(backends)), str(tuning_key)])
    return hashlib.sha256(text.encode()).hexdigest()


class DynamicDispatcher:
    """Callable that routes to the fastest registered backend for each argument signature."""

    _CACHE_FILE = "backend_dispatch.json"

    def __init__(self, fn: Callable, key: List[str], arg_names: List[str], warmup: int = 25, rep: int = 100,
                 use_disk_cache: bool = True, bench_fn: Optional[Callable] = None):
        self._fn = fn
        self._key_names = key
        self._arg_names = arg_names
        self._warmup = warmup
        self._rep = rep
        self._disk = use_disk_cache
        self._bench_fn = bench_fn
        self._backends: Dict[str, Callable] = {}
        self._forced: Optional[str] = None
        self._aliases: Dict[str, str] = {}
        self.cache: Dict[tuple, str] = {}
        self.timings: Dict[tuple, Dict[str, float]] = {}
        self.__name__ = fn.__name__
        self.__doc__ = fn.__doc__

    def register(self, name: str, impl: Callable) -> "DynamicDispatcher":
        self._backends[name] = impl
        return self

    def alias(self, alias: str, name: str) -> "DynamicDispatcher":
        """Let ``force_backend(alias)`` select backend ``name`` (no second timing entry is created)."""
        if name not in self._backends:
            raise KeyError(f"Backend '{name}' not registered in '{self.__name__}'.")
        self._aliases[alias] = name
        return self

    def __call__(self, *args, **kwargs):
        if not self._backends:
            raise RuntimeError(f"[{self.__name__}] No backends registered.")
        if self._forced is not None:
            return self._backends[self._forced](*args, **kwargs)
        key = _tuning_key(self._key_names, args, kwargs, self._arg_names)
        if key not in self.cache:
            self._bench_and_cache(key, args, kwargs)
        return self._backends[self.cache[key]](*args, **kwargs)

    # ------------------------------------------------------------------
    def _timer(self) -> Callable:
        if self._bench_fn is not None:
            return self._bench_fn
        from tritonix_amd.testing import do_bench

        return do_bench

    def _bench_and_cache(self, key: tuple, args: tuple, kwargs: dict) -> None:
        if self._disk and self._load_from_disk(key) is not None:
            return
        timer = self._timer()
        results: Dict[str, float] = {}
        for name, impl in self._backends.items():
            try:
                results[name] = timer(lambda: impl(*args, **kwargs), warmup=self._warmup, rep=self._rep)
            except Exception as exc:  # a failing backend only loses the race
                log.debug("[%s] backend '%s' skipped: %s", self.__name__, name, exc)
        if not results:
            raise RuntimeError(f"[{self.__name__}] All backends failed.")
        winner = min(results, key=results.get)
        log.info("[%s] %s", self.__name__, "  ".join(f"{n}={v:.3f}ms" for n, v in results.items()))
        self.cache[key] = winner
        self.timings[key] = results
        if self._disk:
            self._save_to_disk(key, results, winner)

    def _disk_path(self, key: tuple) -> str:
        return os.path.join(cache_dir(), _disk_key(self.__name__, list(self._backends.keys()), key), self._CACHE_FILE)

    def _load_from_disk(self, key: tuple) -> Optional[str]:
        try:
            path = self._disk_path(key)
            if not os.path.exists(path):
                return None
            with open(path) as f:
                data = json.load(f)
            if data["winner"] not in self._backends:
                return None
            self.cache[key] = data["winner"]
            self.timings[key] = data["timings"]
            return data["winner"]
        except Exception as exc:
            log.debug("[%s] disk miss: %s", self.__name__, exc)
            return None

    def _save_to_disk(self, key: tuple, results: Dict[str, float], winner: str) -> None:
        try:
            path = self._disk_path(key)
            os.makedirs(os.path.dirname(path), exist_ok=True)
            payload = json.dumps({"op": self.__name__, "key": list(key), "winner": winner, "timings": results})
            fd, tmp = tempfile.mkstemp(dir=os.path.dirname(path), suffix=".tmp")
            with os.fdopen(fd, "w") as f:
                f.write(payload)
            os.replace(tmp, path)
        except Exception as exc:
            log.warning("[%s] disk write failed: %s", self.__name__, exc)

    # ------------------------------------------------------------------
    @contextmanager
    def force_backend(self, name: str):
        name = self._aliases.get(name, name)
        if name not in self._backends:
            raise KeyError(f"Backend '{name}' not registered in '{self.__name__}'.")
        self._forced = name
        try:
            yield
        finally:
            self._forced = None

    def clear_cache(self) -> None:
        """Forget the in-memory winners and timings (records on disk stay)."""
        self.cache.clear()
        self.timings.clear()

    def best_config(self) -> Dict[tuple, str]:
        return dict(self.cache)


def dynamic_dispatch(backends: Optional[Dict[str, Callable]] = None, key: Optional[List[str]] = None, warmup: int = 25,
                     rep: int = 100, use_disk_cache: bool = True, bench_fn: Optional[Callable] = None):
    """Build a dispatcher from a ``{name: impl}`` dict, or use as ``@dynamic_dispatch(key=[...])``.

    With a dict the dispatcher takes its name, docstring and argument names
    from the first backend.
    """

    def make(fn: Callable) -> DynamicDispatcher:
        return DynamicDispatcher(fn, key=key or [], arg_names=list(inspect.signature(fn).parameters.keys()),
                                 warmup=warmup, rep=rep, use_disk_cache=use_disk_cache, bench_fn=bench_fn)

    if backends is not None:
        d = make(next(iter(backends.values())))
        for name, impl in backends.items():
            d.register(name, impl)
        return d
    return make
