"""Per-signature choice between interchangeable implementations of one operation.

The first call with a new argument signature times every registered backend
and remembers the winner; later calls go straight to it.  Public surface and
observable behaviour are those of the reference's dispatcher
(tritonix/dispatcher.py:18-35 for the two key functions, :38-145 for the
class, :148-175 for the factory): ``register``, ``force_backend``,
``clear_cache``, ``best_config``, the ``cache`` / ``timings`` dictionaries and
the JSON record ``{"op", "key", "winner", "timings"}`` in a file called
``backend_dispatch.json``.  Differences: records live under
``$TRITONIX_CACHE_DIR`` (default ``~/.cache/tritonix_amd``) rather than in
Triton's cache, the timer is this package's HIP-event ``do_bench`` unless a
``bench_fn`` is injected, ``alias`` lets one backend answer to two names, and a
backend registered with ``raced=False`` is reachable through ``force_backend``
only: it is never timed and never wins a signature (how ``torch.matmul`` stays
available as the correctness oracle without ever serving an unforced call).
"""
from __future__ import annotations

import contextlib
import hashlib
import inspect
import json
import logging
import os
import tempfile
from typing import Any, Callable, Dict, Iterable, List, NamedTuple, Optional, Tuple

__all__ = ["DynamicDispatcher", "dynamic_dispatch", "cache_dir"]

_log = logging.getLogger(__name__)


def cache_dir() -> str:
    """Root of everything this package persists (dispatch records, tuned tile configs)."""
    override = os.environ.get("TRITONIX_CACHE_DIR")
    return override if override else os.path.join(os.path.expanduser("~"), ".cache", "tritonix_amd")


# ---------------------------------------------------------------------------
# signatures
# ---------------------------------------------------------------------------
def _tensor_like(obj: Any) -> bool:
    return all(hasattr(obj, attr) for attr in ("shape", "dtype", "stride"))


def _footprint(obj: Any) -> Tuple:
    """What a tensor contributes to a signature: its extents, then its dtype as text."""
    return (*obj.shape, str(obj.dtype))


def _tuning_key(key_names: List[str], args: tuple, kwargs: dict, arg_names: List[str]) -> tuple:
    """Signature of a call.

    First the keyed arguments in the order the key lists them (a tensor gives
    its footprint, anything else its value; names the call does not bind are
    passed over), then the footprint of every remaining tensor argument in
    binding order: positionals by parameter name, keywords after them.
    """
    call: Dict[str, Any] = {name: value for name, value in zip(arg_names, args)}
    call.update(kwargs)
    sig: List[Any] = []
    for name in key_names:
        if name not in call:
            continue
        value = call[name]
        sig += _footprint(value) if _tensor_like(value) else (value,)
    for name, value in call.items():
        if name not in key_names and _tensor_like(value):
            sig += _footprint(value)
    return tuple(sig)


def _disk_key(op_name: str, backends: Iterable[str], tuning_key: tuple) -> str:
    """Directory name of a record: sha256 over operation, sorted backend names and signature."""
    material = f"{op_name}-{sorted(backends)}-{tuning_key}"
    return hashlib.sha256(material.encode()).hexdigest()


# ---------------------------------------------------------------------------
# records on disk
# ---------------------------------------------------------------------------
class _Verdict(NamedTuple):
    winner: str
    timings: Dict[str, float]


class _RecordStore:
    """One small JSON file per (operation, backend set, signature); unreadable records count as absent."""

    FILE_NAME = "backend_dispatch.json"

    def __init__(self, op_name: str):
        self.op_name = op_name

    def _file(self, backends: Iterable[str], signature: tuple) -> str:
        return os.path.join(cache_dir(), _disk_key(self.op_name, backends, signature), self.FILE_NAME)

    def get(self, backends: Iterable[str], signature: tuple) -> Optional[_Verdict]:
        try:
            with open(self._file(backends, signature)) as fh:
                raw = json.load(fh)
            return _Verdict(raw["winner"], raw["timings"])
        except FileNotFoundError:
            return None
        except (OSError, ValueError, KeyError, TypeError) as err:
            _log.debug("[%s] unusable dispatch record: %s", self.op_name, err)
            return None

    def put(self, backends: Iterable[str], signature: tuple, verdict: _Verdict) -> None:
        target = self._file(backends, signature)
        body = {"op": self.op_name, "key": list(signature), "winner": verdict.winner, "timings": verdict.timings}
        try:
            os.makedirs(os.path.dirname(target), exist_ok=True)
            handle, scratch = tempfile.mkstemp(dir=os.path.dirname(target), suffix=".tmp")
            with os.fdopen(handle, "w") as fh:
                json.dump(body, fh)
            os.replace(scratch, target)          # readers never see a half-written record
        except OSError as err:
            _log.warning("[%s] dispatch record not written: %s", self.op_name, err)


# ---------------------------------------------------------------------------
# the dispatcher
# ---------------------------------------------------------------------------
class DynamicDispatcher:
    """Callable that sends each call to the backend that was fastest for its signature.

    ``cache`` maps signature -> backend name, ``timings`` maps signature ->
    ``{backend: ms}``; both are plain dictionaries a caller may inspect.  One
    ``force_backend`` can be active at a time; the object is not thread-safe.
    """

    def __init__(self, fn: Callable, key: List[str], arg_names: List[str], warmup: int = 25, rep: int = 100,
                 use_disk_cache: bool = True, bench_fn: Optional[Callable] = None):
        self.__name__ = fn.__name__
        self.__doc__ = fn.__doc__
        self._fn = fn
        self._key_names, self._arg_names = key, arg_names
        self._budget = {"warmup": warmup, "rep": rep}
        self._bench_fn = bench_fn
        self._store = _RecordStore(self.__name__) if use_disk_cache else None
        self._backends: Dict[str, Callable] = {}
        self._unraced: set = set()
        self._aliases: Dict[str, str] = {}
        self._forced: Optional[str] = None
        self.cache: Dict[tuple, str] = {}
        self.timings: Dict[tuple, Dict[str, float]] = {}

    # -- registration -------------------------------------------------------
    def register(self, name: str, impl: Callable, raced: bool = True) -> "DynamicDispatcher":
        """Add (or replace) a backend.  ``raced=False`` keeps it out of the timing race and out of ``cache``:
        only ``force_backend(name)`` reaches it."""
        self._backends[name] = impl
        if raced:
            self._unraced.discard(name)
        else:
            self._unraced.add(name)
        return self

    def _contenders(self) -> Dict[str, Callable]:
        return {name: impl for name, impl in self._backends.items() if name not in self._unraced}

    def alias(self, alias: str, name: str) -> "DynamicDispatcher":
        """Make ``force_backend(alias)`` select backend ``name``; timings and records keep the one real name."""
        self._aliases[alias] = self._resolve(name)
        return self

    def _resolve(self, name: str) -> str:
        real = self._aliases.get(name, name)
        if real not in self._backends:
            raise KeyError(f"Backend '{name}' not registered in '{self.__name__}'.")
        return real

    # -- calling ------------------------------------------------------------
    def __call__(self, *args, **kwargs):
        if not self._backends:
            raise RuntimeError(f"[{self.__name__}] No backends registered.")
        if self._forced is not None:
            chosen = self._forced
        else:
            signature = _tuning_key(self._key_names, args, kwargs, self._arg_names)
            chosen = self.cache.get(signature)
            if chosen is None:
                chosen = self._decide(signature, args, kwargs)
        return self._backends[chosen](*args, **kwargs)

    def _decide(self, signature: tuple, args: tuple, kwargs: dict) -> str:
        """Winner for a signature seen for the first time in this process: a record on disk, else a race."""
        names = list(self._backends)
        verdict = self._store.get(names, signature) if self._store else None
        if verdict is None or verdict.winner not in self._contenders():
            verdict = self._race(args, kwargs)
            if self._store:
                self._store.put(names, signature, verdict)
        self.cache[signature], self.timings[signature] = verdict.winner, verdict.timings
        return verdict.winner

    def _race(self, args: tuple, kwargs: dict) -> _Verdict:
        """Time every raced backend on this very call; one that raises simply does not finish."""
        clock = self._bench_fn
        if clock is None:
            from tritonix_amd.testing import do_bench as clock
        finished: Dict[str, float] = {}
        for name, impl in self._contenders().items():
            try:
                finished[name] = clock(lambda: impl(*args, **kwargs), **self._budget)
            except Exception as err:
                _log.debug("[%s] backend '%s' dropped out: %s", self.__name__, name, err)
        if not finished:
            raise RuntimeError(f"[{self.__name__}] All backends failed.")
        _log.info("[%s] %s", self.__name__, ", ".join(f"{n}: {ms:.3f} ms" for n, ms in finished.items()))
        return _Verdict(min(finished, key=finished.__getitem__), finished)

    # -- control ------------------------------------------------------------
    @contextlib.contextmanager
    def force_backend(self, name: str):
        """Inside the block every call goes to ``name`` (or what it aliases); nothing is timed or remembered."""
        self._forced = self._resolve(name)
        try:
            yield
        finally:
            self._forced = None

    def clear_cache(self) -> None:
        """Forget winners and timings held in memory; records on disk stay and are found again."""
        self.cache.clear()
        self.timings.clear()

    def best_config(self) -> Dict[tuple, str]:
        """A copy of signature -> winning backend."""
        return dict(self.cache)


def dynamic_dispatch(backends: Optional[Dict[str, Callable]] = None, key: Optional[List[str]] = None, warmup: int = 25,
                     rep: int = 100, use_disk_cache: bool = True, bench_fn: Optional[Callable] = None):
    """``dynamic_dispatch({"name": impl, ...}, key=[...])`` returns a dispatcher named after the first
    implementation (its docstring and parameter names too); ``@dynamic_dispatch(key=[...])`` on a stub returns an
    empty dispatcher to ``register`` backends on."""

    def wrap(template: Callable) -> DynamicDispatcher:
        params = list(inspect.signature(template).parameters)
        return DynamicDispatcher(template, key=list(key or []), arg_names=params, warmup=warmup, rep=rep,
                                 use_disk_cache=use_disk_cache, bench_fn=bench_fn)

    if backends is None:
        return wrap
    impls = list(backends.items())
    dispatcher = wrap(impls[0][1])
    for name, impl in impls:
        dispatcher.register(name, impl)
    return dispatcher
