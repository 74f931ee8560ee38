"""CPU oracle for the tiled-GEMM path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package; ``tritonix_amd`` never does.

Two layers:

* ``reference_*`` -- what the reference itself checks against: its
  ``"pytorch"`` backend / test oracle is ``torch.matmul``
  (tritonix/ops/matmul.py:291-293, tests/test_matmul.py:15,27), fixed by the
  benchmark contract to an fp32 CPU matmul of the upcast inputs (exact int32
  for int8, via float64) and, for the gated op, ``act(x @ W1) * (x @ W2)`` in
  fp32 (playground/swiglu.py:99-103, playground/fused_glu.py:218-220,296-297).
* ``tiled_*`` -- ctypes bindings of ``gemm_oracle.c``, which walks the
  problem tile by tile and K block by K block like the Triton programs do
  (tritonix/ops/matmul.py:43-108,147-202, tritonix/ops/swiglu.py:24-110).
  Slow; for small shapes.

How each function is pinned (tests/test_oracle.py): ``swizzle2d`` by the 4x4
docstring example the reference holds (playground/swizzle.py:12-25), a ragged
case derived by hand and bijectivity by brute force; ``tiled_matmul`` /
``tiled_splitk`` / ``tiled_matmul_i8`` against float64 / int64 numpy products
and closed forms (identity, all-ones, K-tail shapes); ``splitk_cover`` by the
hand-derived K=100 trace and "every k exactly once"; ``tiled_glu`` by the
closed forms of silu and sigmoid, the identity-gate case reducing to a
product of two plain GEMMs, and the interleave convention; ``reference_*`` are
library routines.  The reference's own tests hold stored vectors for none of
these except the trie (tests/test_trie.py), which tests/test_trie.py here
re-checks.  Split-K, GLU and int8 have no test in the reference at all.

``tiled_conv2d`` (conv_oracle.c) restates conv2d_forward_kernel
(tritonix/ops/conv2d/forward.py:19-165); the reference holds no test or stored
vector for it, so tests/test_conv2d_oracle.py pins it against
``torch.nn.functional.conv2d`` in float64 over asymmetric strides, paddings and
dilations and against closed forms (1x1 filter = matrix product, one-hot filter
= shifted copy, all-ones filter = box sums); ``reference_conv2d`` is that library
routine in fp32.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Tuple

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "liboracle.so")
_lib = None

ACT = {"silu": 1, "sigmoid": 2}


def build() -> str:
    """Compile gemm_oracle.c with gcc (called from __graft_entry__.build and lazily from tests)."""
    subprocess.run(["make", "-s", "-C", HERE], check=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
    return _lib


def _fp(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _es(a) -> Tuple[int, int]:
    return tuple(s // a.itemsize for s in a.strides)


# ---------------------------------------------------------------------------
# index math
# ---------------------------------------------------------------------------
def swizzle2d(i, j, size_i, size_j, size_g):
    oi, oj = ctypes.c_int(), ctypes.c_int()
    lib().oracle_swizzle2d(int(i), int(j), int(size_i), int(size_j), int(size_g), ctypes.byref(oi), ctypes.byref(oj))
    return oi.value, oj.value


def grouped_launch(pid, m, n, block_m, block_n, group_m):
    pm, pn = ctypes.c_int(), ctypes.c_int()
    lib().oracle_grouped_launch(int(pid), int(m), int(n), int(block_m), int(block_n), int(group_m), ctypes.byref(pm),
                                ctypes.byref(pn))
    return pm.value, pn.value


def xcd_remap(pid, total, nxcd=8):
    return int(lib().oracle_xcd_remap(int(pid), int(total), int(nxcd)))


def splitk_cover(k, block_k, split_k):
    cover = np.zeros(k, dtype=np.int32)
    lib().oracle_splitk_cover(ctypes.c_int64(k), int(block_k), int(split_k), _fp(cover))
    return cover


# ---------------------------------------------------------------------------
# tile-walking restatements (small shapes)
# ---------------------------------------------------------------------------
def _i64(*v):
    return [ctypes.c_int64(int(x)) for x in v]


def tiled_matmul(a, b, block_m=32, block_n=32, block_k=16, group_m=4):
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), dtype=np.float32)
    lib().oracle_matmul_f32(_fp(a), _fp(b), _fp(c), *_i64(m, n, k, *_es(a), *_es(b), *_es(c)), int(block_m),
                            int(block_n), int(block_k), int(group_m))
    return c


def tiled_splitk(a, b, split_k, block_m=32, block_n=32, block_k=16, group_m=4):
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), dtype=np.float32)
    lib().oracle_splitk_f32(_fp(a), _fp(b), _fp(c), *_i64(m, n, k, *_es(a), *_es(b), *_es(c)), int(block_m),
                            int(block_n), int(block_k), int(group_m), int(split_k))
    return c


def tiled_matmul_i8(a, b, block_m=32, block_n=32, block_k=32):
    a = np.asarray(a, dtype=np.int8)
    b = np.asarray(b, dtype=np.int8)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), dtype=np.int32)
    lib().oracle_matmul_i8(_fp(a), _fp(b), _fp(c), *_i64(m, n, k, *_es(a), *_es(b), *_es(c)), int(block_m),
                           int(block_n), int(block_k))
    return c


def tiled_glu(x, w12, activation="silu", block_m=32, block_n=32, block_k=16, group_m=4):
    x = np.asarray(x, dtype=np.float32)
    w12 = np.asarray(w12, dtype=np.float32)
    m, k = x.shape
    n = w12.shape[1]
    z = np.empty((m, n // 2), dtype=np.float32)
    lib().oracle_glu_f32(_fp(x), _fp(w12), _fp(z), *_i64(m, n, k, *_es(x), *_es(w12), *_es(z)), int(block_m),
                         int(block_n), int(block_k), int(group_m), int(ACT.get(activation, 0)))
    return z


def conv2d_output_size(h_in, w_in, fh, fw, stride, padding, dilation):
    ho, wo = ctypes.c_int(), ctypes.c_int()
    lib().oracle_conv2d_output_size(int(h_in), int(w_in), int(fh), int(fw), int(stride[0]), int(stride[1]), int(padding[0]),
                                    int(padding[1]), int(dilation[0]), int(dilation[1]), ctypes.byref(ho), ctypes.byref(wo))
    return ho.value, wo.value


def tiled_conv2d(x, w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1), block_m=32, block_n=32, block_k=16):
    """conv_oracle.c on float32 numpy arrays: x [N, C, H, W], w [K, C, R, S], bias [K] or None -> y [N, K, HO, WO] fp32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, c, h, wd = x.shape
    k, c2, r, s = w.shape
    assert c == c2
    ho, wo = conv2d_output_size(h, wd, r, s, stride, padding, dilation)
    assert ho > 0 and wo > 0, "empty output"
    y = np.empty((n, k, ho, wo), dtype=np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    f = lib().oracle_conv2d_f32
    f.restype = ctypes.c_int
    rc = f(_fp(x), _fp(w), None if b is None else _fp(b), _fp(y), n, c, h, wd, k, r, s, int(stride[0]), int(stride[1]),
           int(padding[0]), int(padding[1]), int(dilation[0]), int(dilation[1]), int(block_m), int(block_n), int(block_k))
    assert rc == 0, rc
    return y


# ---------------------------------------------------------------------------
# what the reference checks against: torch CPU, fp32 (exact int32 for int8)
# ---------------------------------------------------------------------------
def reference_conv2d(x, w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1)):
    """``torch.nn.functional.conv2d`` of the upcast inputs in fp32 on the CPU: the reference's own baseline
    (torch_conv2d_forward, tritonix/ops/conv2d/forward.py:314-323)."""
    import torch

    b = None if bias is None else bias.detach().cpu().float()
    return torch.nn.functional.conv2d(x.detach().cpu().float(), w.detach().cpu().float(), b, stride, padding, dilation)



def reference_matmul(a, b):
    """fp32 CPU matmul of the upcast inputs; int8 inputs give the exact int32 product (via float64)."""
    import torch

    a, b = a.detach().cpu(), b.detach().cpu()
    if a.dtype == torch.int8:
        # |sum| <= K * 127^2 stays far below 2^53 for any K that fits in memory: float64 is exact
        return torch.matmul(a.double(), b.double()).to(torch.int32)
    return torch.matmul(a.float(), b.float())


def reference_glu(x, w12, activation="silu"):
    """``act(x @ W1) * (x @ W2)`` in fp32 on the CPU, W1 = even columns of w12, W2 = odd columns."""
    import torch

    x, w12 = x.detach().cpu().float(), w12.detach().cpu().float()
    gate = x @ w12[:, 0::2]
    lin = x @ w12[:, 1::2]
    if activation == "silu":
        gate = torch.nn.functional.silu(gate)
    elif activation == "sigmoid":
        gate = torch.sigmoid(gate)
    return gate * lin


def within_tolerance(out, ref, rel=1e-2):
    """The parity bar for floating-point configs: |out - ref| <= rel*|ref| + rel*rms(ref), plus its summary numbers."""
    import torch

    out, ref = out.detach().cpu().double(), ref.detach().cpu().double()
    rms = ref.pow(2).mean().sqrt()
    err = (out - ref).abs()
    ok = bool((err <= rel * ref.abs() + rel * rms).all())
    return ok, float(err.max()), float(err.max() / ref.abs().max().clamp_min(1e-30))


# ---------------------------------------------------------------------------
# seeded inputs of the five benchmark configurations (generated on the CPU so
# the oracle and the GPU see identical bits)
# ---------------------------------------------------------------------------
CONFIGS = {
    "C1": dict(kind="gemm", dtype="float16", m=1024, n=768, k=512, seed=1),
    "C2": dict(kind="gemm", dtype="bfloat16", m=8192, n=8192, k=8192, seed=2),
    "C3": dict(kind="splitk", dtype="bfloat16", m=16, n=4096, k=14336, seed=3),
    "C4": dict(kind="glu", dtype="bfloat16", m=4096, n=28672, k=4096, seed=4),
    "C5": dict(kind="gemm", dtype="int8", m=8192, n=8192, k=8192, seed=5),
}


def make_inputs(name, scale_down=1):
    """(a, b) CPU tensors of config ``name``; ``scale_down`` divides m, n, k (parity at sizes a CPU finishes fast)."""
    import math

    import torch

    cfg = CONFIGS[name]
    m, n, k = (max(16, cfg[d] // scale_down) for d in ("m", "n", "k"))
    if name == "C3":
        m = cfg["m"]
    g = torch.Generator("cpu").manual_seed(cfg["seed"])
    dt = getattr(torch, cfg["dtype"])
    if name == "C1":
        return torch.randn(m, k, generator=g).to(dt), torch.randn(k, n, generator=g).to(dt)
    if name == "C2":
        s = 1.0 / math.sqrt(k)
        return (torch.randn(m, k, generator=g) * s).to(dt), (torch.randn(k, n, generator=g) * s).to(dt)
    if name == "C3":
        return torch.randn(m, k, generator=g).to(dt), (0.02 * torch.randn(k, n, generator=g)).to(dt)
    if name == "C4":
        x = torch.randn(m, k, generator=g).to(dt)
        w1 = (0.02 * torch.randn(k, n // 2, generator=g)).to(dt)
        w2 = (0.02 * torch.randn(k, n // 2, generator=g)).to(dt)
        return x, torch.stack([w1, w2], dim=2).reshape(k, n).contiguous()
    if name == "C5":
        return (torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8),
                torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8))
    raise KeyError(name)
