"""Timing and resource-error services the tuner and the dispatcher rely on.

The reference takes these from Triton: ``triton.testing.do_bench`` (call sites
tritonix/autotune.py:119,197 and tritonix/dispatcher.py:85) and
``triton.OutOfResources`` (tritonix/autotune.py:6,134).  Here they are small
HIP-event based equivalents with the same call signature and the same
estimate -> warm-up -> repeat protocol (mean of the repeats by default, the
last-level cache flushed before every timed call).
"""
from __future__ import annotations

import statistics
from typing import Callable, List, Optional, Sequence, Union

__all__ = ["do_bench", "OutOfResources", "LDS_LIMIT_BYTES"]

LDS_LIMIT_BYTES = 160 * 1024

# MI355X keeps 256 MiB of Infinity Cache in front of HBM; writing a buffer
# twice that size evicts whatever the benchmarked op left behind.
_FLUSH_BYTES = 512 * 1024 * 1024
_flush_buffers = {}


class OutOfResources(Exception):
    """A kernel configuration needs more of an on-chip resource than exists.

    Same constructor and message as ``triton.OutOfResources(required, limit,
    name)``: the tuner catches it to prune every config that is at least as
    large in each memory parameter.
    """

    def __init__(self, required: int, limit: int, name: str):
        self.required, self.limit, self.name = required, limit, name
        self.message = (f"out of resource: {name}, Required: {required}, Hardware limit: {limit}. "
                        "Reducing block sizes or `num_stages` may help.")
        super().__init__(self.message)

    def __reduce__(self):
        return (type(self), (self.required, self.limit, self.name))


def _flush_buffer(device):
    import torch

    key = (device.type, device.index)
    buf = _flush_buffers.get(key)
    if buf is None:
        buf = torch.empty(_FLUSH_BYTES // 4, dtype=torch.int32, device=device)
        _flush_buffers[key] = buf
    return buf


def _summarize(times: Sequence[float], quantiles, return_mode: str):
    if quantiles is not None:
        import numpy as np

        out = np.quantile(np.asarray(times, dtype=float), list(quantiles)).tolist()
        return out[0] if len(out) == 1 else out
    if return_mode == "all":
        return list(times)
    return {"min": min, "max": max, "mean": statistics.fmean, "median": statistics.median}[return_mode](times)


def do_bench(fn: Callable[[], object], warmup: float = 25, rep: float = 100, grad_to_none=None,
             quantiles: Optional[Sequence[float]] = None, return_mode: str = "mean", flush_cache: bool = True
             ) -> Union[float, List[float]]:
    """Milliseconds one call of ``fn`` takes on the current HIP stream.

    ``warmup`` and ``rep`` are time budgets in milliseconds, not call counts:
    five flushed calls give an estimate, from which the number of warm-up and
    timed calls follows.
    """
    import torch

    if return_mode not in ("min", "max", "mean", "median", "all"):
        raise ValueError(f"unknown return_mode {return_mode!r}")
    if not torch.cuda.is_available():
        raise RuntimeError("do_bench needs a GPU: no HIP device is visible")
    device = torch.device("cuda", torch.cuda.current_device())
    cache = _flush_buffer(device) if flush_cache else None

    fn()
    torch.cuda.synchronize()

    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        if cache is not None:
            cache.zero_()
        fn()
    stop.record()
    torch.cuda.synchronize()
    estimate = start.elapsed_time(stop) / 5
    n_warmup = max(1, int(warmup / estimate)) if estimate > 0 else 1
    n_repeat = max(1, int(rep / estimate)) if estimate > 0 else 1

    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    stops = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for _ in range(n_warmup):
        fn()
    for i in range(n_repeat):
        if grad_to_none is not None:
            for x in grad_to_none:
                x.grad = None
        if cache is not None:
            cache.zero_()
        starts[i].record()
        fn()
        stops[i].record()
    torch.cuda.synchronize()
    times = [s.elapsed_time(e) for s, e in zip(starts, stops)]
    return _summarize(times, quantiles, return_mode)
