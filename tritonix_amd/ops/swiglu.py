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

__all__ = ["glu_kernel", "glu", "swiglu", "swiglu_ffn", "fused_glu", "silu", "interleave_weights"]

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
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"glu is built for float16 and bfloat16, got {x.dtype}")
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
