"""Launch objects that keep the reference's Triton calling convention over the HIP engine.

A reference kernel is launched as ``kernel[grid](a, b, c, m, n, k, stride_am,
stride_ak, stride_bk, stride_bn, stride_cm, stride_cn, block_m=..., block_n=...,
block_k=..., group_m=..., [split_k=...,] num_stages=..., num_warps=...)``
(tritonix/ops/matmul.py:222-236, :249-263; the GLU kernel adds ``use_tf32``
and ``activation``, tritonix/ops/swiglu.py:24-43).  ``HipKernel`` accepts the
same call, turns it into one ``tnx_gemm`` through the C ABI and launches on
torch's current stream.  ``grid`` is accepted for compatibility; the engine
derives its own 1-D grid from the shape and the tile.
"""
from __future__ import annotations

import ctypes
from collections import OrderedDict
from typing import Callable, List, Optional, Tuple

from tritonix_amd import _C

__all__ = ["HipKernel", "cdiv"]


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


_POSITIONAL = ("a", "b", "c", "m", "n", "k", "stride_am", "stride_ak", "stride_bk", "stride_bn", "stride_cm",
               "stride_cn")
_ACTIVATIONS = {"silu": _C.EPI_GLU_SILU, "sigmoid": _C.EPI_GLU_SIGMOID}

# split-K scratch buffers, most recently used last; at most _MAX_WORKSPACES are kept alive
_workspaces: "OrderedDict[Tuple[int, int], object]" = OrderedDict()
_MAX_WORKSPACES = 8


def _torch_dtype_code(dtype) -> int:
    import torch

    table = {torch.float16: _C.F16, torch.bfloat16: _C.BF16, torch.int8: _C.I8, torch.int32: _C.I32,
             torch.float32: _C.F32}
    if dtype not in table:
        raise ValueError(f"dtype {dtype} has no HIP kernel (float16, bfloat16, int8 and -- as a bf16 split -- float32 inputs are built)")
    return table[dtype]


def out_dtype_for(dtype):
    """Output dtype of the engine for an input dtype: floats keep theirs, int8 accumulates to int32."""
    import torch

    return torch.int32 if dtype == torch.int8 else dtype


def _workspace_key(device, stream_ptr: int, atomic: bool = False) -> Tuple[int, int, bool]:
    import torch

    return (device.index if device.index is not None else torch.cuda.current_device(), stream_ptr, bool(atomic))


def _workspace(device, stream_ptr: int, nbytes: int, atomic: bool = False):
    """Split-K scratch, one growing buffer per (device, stream), the least recently used ones released.

    Allocated zero-filled: the leading counter region must start at zero and every launch leaves it zero.  A
    launch that fails part-way may leave counters set, so ``drop_workspace`` forgets the buffer after any error
    and the next launch starts from a freshly zeroed one.
    """
    import torch

    # launches that reduce with atomics need their sum region zero and leave it zero; ordered launches leave
    # slices behind: the two modes never share a buffer
    key = _workspace_key(device, stream_ptr, atomic)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    _workspaces.move_to_end(key)
    if _capturing():
        # A launch recorded into a HIP graph bakes this pointer into the graph: the buffer must outlive every
        # replay, so it is never released (not by the eviction below, not when a later call needs a larger one).
        if not any(kept is buf for kept in _captured_workspaces):
            _captured_workspaces.append(buf)
        return buf
    while len(_workspaces) > _MAX_WORKSPACES:
        _workspaces.popitem(last=False)       # launches already enqueued keep their buffer alive through the allocator's stream ordering
    return buf


# scratch buffers handed to launches that were recorded into a HIP graph: alive until the process ends
_captured_workspaces: list = []


def _capturing() -> bool:
    import torch

    try:
        return bool(torch.cuda.is_current_stream_capturing())
    except (RuntimeError, AssertionError):
        return False


def drop_workspace(device, stream_ptr: int) -> None:
    """Forget the scratch of (device, stream): called when a launch on it reported an error."""
    for atomic in (False, True):
        _workspaces.pop(_workspace_key(device, stream_ptr, atomic), None)


def split_f32_operands(bound: dict, stream: int) -> dict:
    """A bound float32 call rewritten as the bf16 call that computes it.

    The reference's kernels take float32 operands and multiply them in TF32 (tritonix/ops/matmul.py:98,
    tritonix/ops/swiglu.py:89-93); gfx950 has no TF32 matrix instruction.  ``tnx_split_f32`` cuts each operand into a
    bf16 head and a bf16 tail and lays out ``[hi | hi | lo]`` along the columns of A and ``[hi ; lo ; hi]`` along the
    rows of B, so one bf16 GEMM with ``k' = 3k`` and an fp32 result is ``hi(a) hi(b) + hi(a) lo(b) + lo(a) hi(b)``: error
    O(2^-16) per product, below TF32's.  The two scratch operands are contiguous, whatever strides the call had.
    """
    import torch

    a, b = bound["a"], bound["b"]
    m, n, k = int(bound["m"]), int(bound["n"]), int(bound["k"])
    lib = _C.load()
    a3 = torch.empty((m, 3 * k), dtype=torch.bfloat16, device=a.device)
    b3 = torch.empty((3 * k, n), dtype=torch.bfloat16, device=a.device)
    for src, rows, cols, sr, sc, dst, side in ((a, m, k, bound["stride_am"], bound["stride_ak"], a3, 0),
                                               (b, k, n, bound["stride_bk"], bound["stride_bn"], b3, 1)):
        status = lib.tnx_split_f32(src.data_ptr(), rows, cols, int(sr), int(sc), dst.data_ptr(), side, stream)
        if status != _C.OK:
            raise RuntimeError(f"tnx_split_f32: {_C.strerror(status)}")
    out = dict(bound)
    out.update(a=a3, b=b3, k=3 * k, stride_am=3 * k, stride_ak=1, stride_bk=n, stride_bn=1)
    return out


class _BoundLaunch:
    def __init__(self, kernel: "HipKernel", grid):
        self.kernel, self.grid = kernel, grid

    def __call__(self, *args, **kwargs):
        return self.kernel.run(*args, grid=self.grid, **kwargs)


class HipKernel:
    """One entry of the HIP engine behind the Triton launch protocol."""

    def __init__(self, name: str, tile_params: List[str], glu: bool = False, doc: Optional[str] = None):
        self.__name__ = name
        self.__doc__ = doc
        self.tile_params = list(tile_params)
        self.glu = glu
        # optional keywords after the reference's own: a K split for kernels whose signature has none, the
        # number of trailing tiles the split applies to (0 = all), and the two scheduling switches of the engine
        # (persistent: one workgroup per CU walks its tiles; superblock: 16x16 super-block launch order)
        # atomic_reduce: split-K slices are added into one fp32 copy with atomics instead of being summed in order
        self.optional = [n for n in ("split_k", "tail_tiles", "persistent", "superblock", "atomic_reduce")
                         if n not in self.tile_params]
        self.arg_names = (list(_POSITIONAL) + self.tile_params + (["use_tf32", "activation"] if glu else [])
                          + self.optional)
        self.pre_run_hooks: List[Callable] = []
        self.specialize_keys: List[str] = []

    def __getitem__(self, grid) -> _BoundLaunch:
        return _BoundLaunch(self, grid)

    def add_pre_run_hook(self, hook: Callable) -> None:
        """``hook(*args, **kwargs)`` runs before every launch, as with a Triton ``JITFunction``."""
        self.pre_run_hooks.append(hook)

    # ------------------------------------------------------------------
    def _bind(self, args, kwargs) -> dict:
        if len(args) > len(self.arg_names):
            raise TypeError(f"{self.__name__} takes at most {len(self.arg_names)} arguments, got {len(args)}")
        bound = dict(zip(self.arg_names, args))
        for k, v in kwargs.items():
            if k not in self.arg_names:
                raise TypeError(f"{self.__name__} got an unexpected keyword argument '{k}'")
            if k in bound:
                raise TypeError(f"{self.__name__} got multiple values for argument '{k}'")
            bound[k] = v
        missing = [n for n in list(_POSITIONAL) + self.tile_params if n not in bound]
        if missing:
            raise TypeError(f"{self.__name__} missing arguments: {', '.join(missing)}")
        return bound

    def make_args(self, bound: dict) -> _C.GemmArgs:
        """Fill a ``tnx_gemm_args`` from a bound call (pointers from the tensors' ``data_ptr``)."""
        a, b, c = bound["a"], bound["b"], bound["c"]
        g = _C.GemmArgs()
        g.a, g.b, g.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
        g.m, g.n, g.k = int(bound["m"]), int(bound["n"]), int(bound["k"])
        g.stride_am, g.stride_ak = int(bound["stride_am"]), int(bound["stride_ak"])
        g.stride_bk, g.stride_bn = int(bound["stride_bk"]), int(bound["stride_bn"])
        g.stride_cm, g.stride_cn = int(bound["stride_cm"]), int(bound["stride_cn"])
        g.in_dtype = _torch_dtype_code(a.dtype)
        if b.dtype != a.dtype:
            raise ValueError(f"a and b must share a dtype, got {a.dtype} and {b.dtype}")
        g.out_dtype = _torch_dtype_code(c.dtype)
        g.block_m, g.block_n, g.block_k = int(bound["block_m"]), int(bound["block_n"]), int(bound["block_k"])
        g.group_m = int(bound["group_m"])
        g.split_k = int(bound.get("split_k", 1))
        g.tail_tiles = int(bound.get("tail_tiles", 0))
        g.schedule = ((_C.SCHED_PERSISTENT if int(bound.get("persistent", 0)) else 0)
                      | (_C.SCHED_SUPERBLOCK if int(bound.get("superblock", 0)) else 0)
                      | (_C.SCHED_ATOMIC_REDUCE if int(bound.get("atomic_reduce", 0)) else 0))
        g.num_stages, g.num_warps = int(bound["num_stages"]), int(bound["num_warps"])
        if self.glu:
            # "silu" and "sigmoid" gate explicitly; like the reference kernel, any other
            # value leaves the gate un-activated (tritonix/ops/swiglu.py:100-102)
            g.epilogue = _ACTIVATIONS.get(bound.get("activation", "silu"), _C.EPI_GLU_IDENTITY)
        else:
            g.epilogue = _C.EPI_NONE
        return g

    def run(self, *args, grid=None, **kwargs):
        import torch

        bound = self._bind(args, kwargs)
        a, b, c = bound["a"], bound["b"], bound["c"]
        for name, t in (("a", a), ("b", b), ("c", c)):
            if not isinstance(t, torch.Tensor) or not t.is_cuda:
                raise ValueError(f"{self.__name__}: '{name}' must be a tensor on a HIP device")
        if not (a.device == b.device == c.device):
            raise ValueError(f"{self.__name__}: a, b and c must live on one device")
        if grid is not None and not callable(grid):
            if not all(isinstance(g, int) and g >= 0 for g in tuple(grid)):
                raise ValueError(f"{self.__name__}: grid must be a tuple of non-negative ints, got {grid!r}")
        for hook in self.pre_run_hooks:
            hook(*args, **kwargs)

        lib = _C.load()
        if a.dtype == torch.float32 and b.dtype == torch.float32:
            if c.dtype != torch.float32:
                raise ValueError(f"{self.__name__}: float32 operands give a float32 result, got c of {c.dtype}")
            with torch.cuda.device(a.device):
                bound = split_f32_operands(bound, torch.cuda.current_stream(a.device).cuda_stream)
        g = self.make_args(bound)
        if a.device.index != torch.cuda.current_device():
            with torch.cuda.device(a.device):
                status = self._launch(lib, g, a.device)
        else:
            status = self._launch(lib, g, a.device)
        _C.raise_for_status(status, g)
        return None

    @staticmethod
    def _launch(lib, g, device) -> int:
        import torch

        stream = torch.cuda.current_stream(device).cuda_stream
        g.stream = stream
        if g.split_k > 1:
            need = int(lib.tnx_gemm_workspace_bytes(ctypes.byref(g)))
            if need:
                ws = _workspace(device, stream, need, bool(g.schedule & _C.SCHED_ATOMIC_REDUCE))
                g.workspace, g.workspace_bytes = ws.data_ptr(), ws.numel()
        status = lib.tnx_gemm(ctypes.byref(g))
        if status == _C.E_HIP and g.split_k > 1:
            drop_workspace(device, stream)
        return status

    def prepare(self, *args, **kwargs) -> Callable[[], None]:
        """Bind a launch once and return a zero-argument callable that repeats it.

        The tensors, tile config, stream and split-K workspace are captured at bind time; the returned
        callable only performs the C-ABI call (for launch-bound shapes and for benchmarks).
        """
        import torch

        bound = self._bind(args, kwargs)
        lib = _C.load()
        if bound["a"].dtype == torch.float32:
            raise ValueError(f"{self.__name__}.prepare binds 16-bit and int8 launches; a float32 call splits its operands "
                             "on every launch")
        g = self.make_args(bound)
        device = bound["a"].device
        stream = torch.cuda.current_stream(device).cuda_stream
        g.stream = stream
        keep = [bound["a"], bound["b"], bound["c"]]
        if g.split_k > 1:
            need = int(lib.tnx_gemm_workspace_bytes(ctypes.byref(g)))
            ws = _workspace(device, stream, need, bool(g.schedule & _C.SCHED_ATOMIC_REDUCE))
            g.workspace, g.workspace_bytes = ws.data_ptr(), ws.numel()
            keep.append(ws)
        status = lib.tnx_gemm_supported(ctypes.byref(g))
        _C.raise_for_status(status, g)
        ref, fn = ctypes.byref(g), lib.tnx_gemm

        def launch(_keep=keep, _g=g):
            st = fn(ref)
            if st:
                if _g.split_k > 1:
                    drop_workspace(device, stream)
                _C.raise_for_status(st, _g)

        return launch

    # host-only helpers -------------------------------------------------
    def lds_bytes(self, in_dtype_code: int, block_m: int, block_n: int, block_k: int, num_stages: int,
                  num_warps: int = 4, persistent: int = 0) -> int:
        """LDS bytes per workgroup of a tile config (no GPU needed)."""
        g = _C.GemmArgs()
        g.in_dtype = in_dtype_code
        g.block_m, g.block_n, g.block_k, g.num_stages, g.num_warps = block_m, block_n, block_k, num_stages, num_warps
        g.schedule = _C.SCHED_PERSISTENT if persistent else 0
        return int(_C.load().tnx_gemm_lds_bytes(ctypes.byref(g)))

    def __repr__(self):
        return f"<HipKernel {self.__name__}>"
