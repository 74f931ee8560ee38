"""Fused GLU / SwiGLU up-projection: ``z = act(x @ W1) * (x @ W2)`` in one GEMM pass.

``w12`` holds W1 and W2 interleaved column-wise -- W1 in the even columns
(the gate), W2 in the odd ones -- so the gate/linear pair of an output element
lands in one lane of the MFMA result and the gating is applied in the
epilogue, before anything is written.  Kernel contract follows
tritonix/ops/swiglu.py:24-110 of the reference (``glu_kernel``; phase 1 of
``swiglu_kernel`` :155-205 is the same computation); the interleave convention
is the one of playground/fused_glu.py:243,296-297.  The reference ships no
host wrapper for it; ``glu`` / ``swiglu`` / ``fused_glu`` below are modelled on
playground/fused_glu.py:147-176 (``fused_glu(a, b) -> c[M, N//2]``).

Activations: ``"silu"`` (SwiGLU) and ``"sigmoid"`` (classic GLU) are applied
explicitly.  Any other value leaves the gate un-activated (bilinear), which
is what the reference kernel does for every value but ``"silu"``
(tritonix/ops/swiglu.py:100-102).
"""
from __future__ import annotations

import torch

from tritonix_amd.autotune import Choice, PowerOfTwo, Range, tunable
from tritonix_amd.kernel import HipKernel, cdiv
import importlib

_mm = importlib.import_module("tritonix_amd.ops.matmul")  # the module: the package attribute `matmul` is the dispatcher

__all__ = ["glu_kernel", "swiglu_kernel", "glu", "swiglu", "swiglu_ffn", "fused_glu", "silu", "interleave_weights"]

glu_kernel = tunable(
    keys=["m", "n", "k"],
    space={
        "block_m": PowerOfTwo(64, 256),
        "block_n": PowerOfTwo(64, 256),
        "block_k": PowerOfTwo(32, 128),
        "group_m": Choice([4, 8]),
        "num_stages": Range(2, 4),
        "num_warps": Choice([4, 8]),
    },
    memory_params={"block_m", "block_n", "block_k", "num_stages"},
)(HipKernel("glu_kernel", ["block_m", "block_n", "block_k", "group_m", "num_stages", "num_warps"], glu=True,
            doc="Z = act(X @ W12[:, 0::2]) * (X @ W12[:, 1::2]); n is the interleaved width, Z has n/2 columns"))


class _FeedForwardLaunch:
    def __init__(self, kernel, grid):
        self.kernel, self.grid = kernel, grid

    def __call__(self, *args, **kwargs):
        return self.kernel.run(*args, grid=self.grid, **kwargs)


class SwigluKernel:
    """``swiglu_kernel`` of the reference as a launch object over the HIP engine.

    Calling convention of tritonix/ops/swiglu.py:127-152: ``swiglu_kernel[grid](x, w12, w3, z, m, n, k, f,
    stride_xm, stride_xk, stride_wk, stride_wn, stride_w3n, stride_w3l, stride_zm, stride_zl, block_m=...,
    block_n=..., block_k=..., group_m=..., block_l=..., use_tf32=True, activation="silu", num_stages=...,
    num_warps=...)`` with ``x[m, k]``, the interleaved ``w12[k, n]`` (gate in the even columns), ``w3[n/2, f]`` and
    ``z[m, f]``.  It computes ``z = (act(x @ W1) * (x @ W2)) @ w3``.

    The reference's body is a draft that was never launched (its phase 2, :207-230, adds a ``block_m x f`` tile
    into ``z`` with atomics from every column tile and has index errors); what it is meant to compute is
    playground/swiglu.py:99-103.  Here phase 1 (:155-205) is one launch of the gated tile kernel -- ``block_m x
    block_n x block_k`` tiles, the gate applied in the epilogue -- into an ``[m, n/2]`` intermediate of the input
    dtype, and phase 2 one launch of the tile kernel with ``block_m x block_l x block_k`` tiles on that
    intermediate and ``w3``; ``z`` is written, not accumulated into, and needs no zero fill.  ``use_tf32`` is
    accepted and has no effect on 16-bit inputs, as in the reference (:89-93).
    """

    _POSITIONAL = ("x", "w12", "w3", "z", "m", "n", "k", "f", "stride_xm", "stride_xk", "stride_wk", "stride_wn",
                   "stride_w3n", "stride_w3l", "stride_zm", "stride_zl")
    tile_params = ["block_m", "block_n", "block_k", "group_m", "block_l", "num_stages", "num_warps"]

    def __init__(self):
        self.__name__ = "swiglu_kernel"
        self.__doc__ = "Z = (act(X @ W12[:, 0::2]) * (X @ W12[:, 1::2])) @ W3"
        self.arg_names = list(self._POSITIONAL) + ["block_m", "block_n", "block_k", "group_m", "block_l", "use_tf32",
                                                   "activation", "num_stages", "num_warps"]
        self.pre_run_hooks = []
        self.specialize_keys = []

    def __getitem__(self, grid):
        return _FeedForwardLaunch(self, grid)

    def add_pre_run_hook(self, hook) -> None:
        self.pre_run_hooks.append(hook)

    def _bind(self, args, kwargs) -> dict:
        if len(args) > len(self.arg_names):
            raise TypeError(f"swiglu_kernel takes at most {len(self.arg_names)} arguments, got {len(args)}")
        bound = dict(zip(self.arg_names, args))
        for name, value in kwargs.items():
            if name not in self.arg_names:
                raise TypeError(f"swiglu_kernel got an unexpected keyword argument '{name}'")
            if name in bound:
                raise TypeError(f"swiglu_kernel got multiple values for argument '{name}'")
            bound[name] = value
        missing = [name for name in list(self._POSITIONAL) + self.tile_params if name not in bound]
        if missing:
            raise TypeError(f"swiglu_kernel missing arguments: {', '.join(missing)}")
        return bound

    def run(self, *args, grid=None, **kwargs):
        b = self._bind(args, kwargs)
        x, w12, w3, z = b["x"], b["w12"], b["w3"], b["z"]
        m, n, k, f = int(b["m"]), int(b["n"]), int(b["k"]), int(b["f"])
        if n % 2:
            raise ValueError("the interleaved weight must have an even number of columns")
        for hook in self.pre_run_hooks:
            hook(*args, **kwargs)
        # phase 1: gated up-projection into the intermediate (input dtype, row-major)
        h = torch.empty((m, n // 2), device=x.device, dtype=x.dtype)
        ring = dict(num_stages=int(b["num_stages"]), num_warps=int(b["num_warps"]))
        glu_kernel[(cdiv(m, b["block_m"]), cdiv(n, b["block_n"]))](
            x, w12, h, m, n, k, b["stride_xm"], b["stride_xk"], b["stride_wk"], b["stride_wn"], h.stride(0), h.stride(1),
            block_m=b["block_m"], block_n=b["block_n"], block_k=b["block_k"], group_m=b["group_m"],
            use_tf32=b.get("use_tf32", True), activation=b.get("activation", "silu"), **ring)
        # phase 2: down-projection, block_l columns of z per tile
        _mm.matmul_kernel[(cdiv(m, b["block_m"]), cdiv(f, b["block_l"]))](
            h, w3, z, m, f, n // 2, h.stride(0), h.stride(1), b["stride_w3n"], b["stride_w3l"], b["stride_zm"], b["stride_zl"],
            block_m=b["block_m"], block_n=b["block_l"], block_k=b["block_k"], group_m=b["group_m"], **ring)
        return None

    def __repr__(self):
        return "<SwigluKernel swiglu_kernel>"


swiglu_kernel = tunable(
    keys=["m", "n", "k"],
    space={
        "block_m": PowerOfTwo(64, 256),
        "block_n": PowerOfTwo(64, 256),
        "block_k": PowerOfTwo(32, 128),
        "block_l": PowerOfTwo(64, 256),
        "group_m": Choice([4, 8]),
        "num_stages": Range(2, 4),
        "num_warps": Choice([4, 8]),
    },
    memory_params={"block_m", "block_n", "block_k", "block_l", "num_stages"},
)(SwigluKernel())


def silu(x: torch.Tensor) -> torch.Tensor:
    return torch.sigmoid(x) * x


def interleave_weights(w1: torch.Tensor, w2: torch.Tensor) -> torch.Tensor:
    """[K, N] gate and linear weights -> one [K, 2N] matrix, gate in the even columns."""
    if w1.shape != w2.shape:
        raise ValueError(f"w1 and w2 must have one shape, got {tuple(w1.shape)} and {tuple(w2.shape)}")
    return torch.stack([w1, w2], dim=2).reshape(w1.shape[0], 2 * w1.shape[1]).contiguous()


def _launch_glu(x, w12, cfg, activation):
    m, k = x.shape
    _, n = w12.shape
    z = torch.empty((m, n // 2), device=x.device, dtype=x.dtype)
    grid = (cdiv(m, cfg["block_m"]), cdiv(n, cfg["block_n"]))
    glu_kernel[grid](x, w12, z, m, n, k, x.stride(0), x.stride(1), w12.stride(0), w12.stride(1), z.stride(0),
                     z.stride(1), activation=activation, **cfg)
    return z


_glu_cfg = {}


def glu(x: torch.Tensor, w12: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """``act(x @ w12[:, 0::2]) * (x @ w12[:, 1::2])`` -> ``[m, n/2]``, tile config tuned once per shape."""
    if x.dim() != 2 or w12.dim() != 2 or x.shape[1] != w12.shape[0]:
        raise ValueError(f"glu expects x[m,k] and w12[k,2n], got {tuple(x.shape)} and {tuple(w12.shape)}")
    if w12.shape[1] % 2:
        raise ValueError("the interleaved weight must have an even number of columns")
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise ValueError(f"glu is built for float16, bfloat16 and float32, got {x.dtype}")
    x, w12 = _mm.dma_operands(x, w12)
    m, k = x.shape
    n = w12.shape[1]
    key = (m, n, k, x.dtype, _mm.dma_layout(x, w12))
    return _mm.run_memoised(_glu_cfg, "glu", key, glu_kernel, lambda cfg: _launch_glu(x, w12, cfg, activation),
                            lambda: _mm.default_config(x, w12))


def swiglu(x: torch.Tensor, w12: torch.Tensor) -> torch.Tensor:
    """SwiGLU up-projection: ``silu(x @ W1) * (x @ W2)`` with ``w12`` the interleaved ``[W1 | W2]``."""
    return glu(x, w12, activation="silu")


def swiglu_ffn(x: torch.Tensor, w12: torch.Tensor, w3: torch.Tensor, activation: str = "silu") -> torch.Tensor:
    """SwiGLU feed-forward block ``(act(x @ W1) * (x @ W2)) @ W3``.

    What the reference's draft ``swiglu_kernel`` is meant to compute (tritonix/ops/swiglu.py:127-230;
    playground/swiglu.py:99-103).  The draft fuses the down-projection into the same kernel with atomic
    adds and was never launched; here the gated up-projection is the fused GLU kernel and the
    down-projection is the tiled GEMM, two launches with the [m, n] intermediate in the input dtype.
    """
    if w3.dim() != 2 or w3.shape[0] != w12.shape[1] // 2:
        raise ValueError(f"w3 must be [{w12.shape[1] // 2}, f], got {tuple(w3.shape)}")
    return _mm.triton_matmul(glu(x, w12, activation=activation), w3)


def fused_glu(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Name used by the reference's playground wrapper: SiLU-gated GLU, ``c[M, N//2]``."""
    return glu(a, b, activation="silu")
