"""Dense GEMM ops: ``matmul`` (dispatcher), ``triton_matmul`` (tuned tiled GEMM), ``matmul_splitk``.

Public surface and launch flow follow tritonix/ops/matmul.py of the reference:
the ``@tunable`` kernels ``matmul_kernel`` (:30-108) and ``gemm_splitk_kernel``
(:133-202), the host launchers ``_launch_matmul`` (:217-237) and
``_launch_splitk`` (:240-264), the per-shape config memo and ``triton_matmul``
/ ``matmul_splitk`` (:267-288) and the dispatcher instance ``matmul``
(:291-293).  The kernels behind them are the gfx950 HIP tile kernels of
libtritonix_hip.so; ``torch.matmul`` stays registered as the ``"pytorch"``
backend and serves as the correctness oracle, exactly as in the reference.

Deliberate differences:
  * tile spaces are the ones that exist as HIP kernels (64..256 tiles, 2..4
    LDS stages); a combination that is not built raises ``ValueError`` and the
    tuner skips it, one that exceeds 160 KiB of LDS raises ``OutOfResources``
    before any launch and the trie prunes above it;
  * the config memo is keyed by dtype and by the layout class of the operands
    (row-major, 16-byte aligned rows and base pointers, or anything else) as
    well as (m, n, k): one process runs f16, bf16 and int8 problems, and most
    tiles exist only with the direct-to-LDS loader that needs the first class;
  * ``matmul`` keeps the backend names "triton" and "pytorch"; only "triton" (the
    HIP engine, which settles tile against K split in its own config memo) is
    timed, ``torch.matmul`` is registered un-raced, for ``force_backend``;
  * int8 inputs give an int32 result; float32 inputs run as a three-term bf16 split with an fp32 result
    (``tritonix_amd.kernel.split_f32_operands``) where the reference multiplies them in TF32;
  * split-K sums fp32 partials from a workspace and rounds once, where the
    reference rounds each partial to the output dtype and adds atomically
    (tritonix/ops/matmul.py:195-202); the ``_zero_output`` hook is gone with it.
"""
from __future__ import annotations

import os

import torch

from tritonix_amd.autotune import Choice, PowerOfTwo, Range, tunable
from tritonix_amd.dispatcher import dynamic_dispatch
from tritonix_amd.kernel import HipKernel, cdiv, out_dtype_for

__all__ = ["matmul", "triton_matmul", "hip_matmul", "matmul_splitk", "matmul_skinny", "matmul_kernel", "gemm_splitk_kernel",
           "dma_layout", "dma_operands", "run_memoised",
           "swizzle2d", "grouped_launch", "TUNE_OPTIONS", "load_tuned", "save_tuned"]

# keyword arguments handed to ``.tune`` on a config-memo miss (tests shrink the time budgets)
TUNE_OPTIONS = {"warmup": 25, "rep": 100}

_TILE = ["block_m", "block_n", "block_k", "group_m", "num_stages", "num_warps"]

matmul_kernel = tunable(
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
)(HipKernel("matmul_kernel", _TILE, doc="C = A x B. A has shape (M, K), B has shape (K, N) and C has shape (M, N)"))

gemm_splitk_kernel = tunable(
    keys=["m", "n", "k"],
    space={
        "block_m": PowerOfTwo(16, 128),
        "block_n": PowerOfTwo(32, 256),
        "block_k": PowerOfTwo(32, 128),
        "group_m": Choice([4, 8]),
        "split_k": PowerOfTwo(2, 16),
        "num_stages": Range(2, 6),
        "num_warps": Choice([4, 8]),
    },
    memory_params={"block_m", "block_n", "block_k", "num_stages"},
)(HipKernel("gemm_splitk_kernel", ["block_m", "block_n", "block_k", "group_m", "split_k", "num_stages", "num_warps"],
            doc="C = A x B with K cut into split_k slices; fp32 partials, one rounding"))


def swizzle2d(i, j, size_i, size_j, size_g):
    """Tile-id remap the kernels apply: rows of tiles are walked in groups of ``size_g``, column-major inside a group.

    Same mapping as ``tl.swizzle2d`` (called at tritonix/ops/matmul.py:70); host-side copy for tests and tooling.
    """
    ij = i * size_j + j
    per_group = size_g * size_j
    first_row = (ij // per_group) * size_g
    rows = min(size_i - first_row, size_g)
    r = ij % per_group
    return first_row + r % rows, r // rows


def grouped_launch(pid, m, n, block_m, block_n, group_m):
    """1-D program id -> (pid_m, pid_n) in grouped order.

    Same intent as the reference's unused helper (tritonix/ops/matmul.py:111-130) but computed with the
    ``swizzle2d`` formula, which stays a bijection when the last group of tile rows is ragged.
    """
    grid_m, grid_n = cdiv(m, block_m), cdiv(n, block_n)
    return swizzle2d(pid // grid_n, pid % grid_n, grid_m, grid_n, group_m)


def _check_2d(a, b):
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError(f"matmul expects 2-D tensors, got {tuple(a.shape)} and {tuple(b.shape)}")
    if a.shape[1] != b.shape[0]:
        raise ValueError(f"inner dimensions differ: {tuple(a.shape)} @ {tuple(b.shape)}")


def _launch_matmul(a, b, cfg):
    m, k = a.shape
    _, n = b.shape
    c = torch.empty((m, n), device=a.device, dtype=out_dtype_for(a.dtype))
    grid = (cdiv(m, cfg["block_m"]), cdiv(n, cfg["block_n"]))
    matmul_kernel[grid](a, b, c, m, n, k, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1),
                        **cfg)
    return c


def _launch_splitk(a, b, cfg):
    m, k = a.shape
    _, n = b.shape
    # no zero fill: the kernel owns its workspace and writes every element of c
    c = torch.empty((m, n), device=a.device, dtype=out_dtype_for(a.dtype))
    grid = (cdiv(m, cfg["block_m"]), cdiv(n, cfg["block_n"]), cfg["split_k"])
    gemm_splitk_kernel[grid](a, b, c, m, n, k, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0),
                             c.stride(1), **cfg)
    return c


_matmul_cfg = {}
_splitk_cfg = {}


# ---------------------------------------------------------------------------
# tuned tile configs on disk.  The reference only persists the dispatcher's backend winner
# (tritonix/dispatcher.py:100-128) and re-tunes every process; here the tile config a grid
# search picked is written next to it, one small JSON file per (op, shape, dtype).
# ---------------------------------------------------------------------------
def _tuned_path(op: str, key: tuple) -> str:
    import hashlib

    from tritonix_amd.dispatcher import cache_dir

    digest = hashlib.sha256(f"{op}-{key}".encode()).hexdigest()
    return os.path.join(cache_dir(), "tuned", digest + ".json")


def load_tuned(op: str, key: tuple):
    """Tile config stored for (op, key), or None.  ``TRITONIX_TUNE_CACHE=0`` switches the store off."""
    import json

    if os.environ.get("TRITONIX_TUNE_CACHE", "1") in ("0", "false", "False"):
        return None
    try:
        with open(_tuned_path(op, key)) as f:
            rec = json.load(f)
        if rec.get("op") == op and rec.get("key") == [str(k) for k in key] and isinstance(rec.get("config"), dict):
            return {k: int(v) for k, v in rec["config"].items()}
    except (OSError, ValueError, TypeError):
        pass
    return None


def save_tuned(op: str, key: tuple, cfg: dict) -> None:
    import json
    import tempfile

    if os.environ.get("TRITONIX_TUNE_CACHE", "1") in ("0", "false", "False"):
        return
    try:
        path = _tuned_path(op, key)
        os.makedirs(os.path.dirname(path), exist_ok=True)
        fd, tmp = tempfile.mkstemp(dir=os.path.dirname(path), suffix=".tmp")
        with os.fdopen(fd, "w") as f:
            json.dump({"op": op, "key": [str(k) for k in key], "config": cfg}, f)
        os.replace(tmp, path)
    except OSError:
        pass


def dma_layout(a, b) -> int:
    """Layout class of the operands, part of every config-memo key: 1 = row-major A and B, 2 = row-major A and
    k-contiguous B (``w.t()`` of a row-major weight), both with 16-byte aligned rows and base pointers -- the two
    layouts the direct-to-LDS loaders take as they are; 3, 4 = the same two layouts as they take them with the last K
    slab loaded chunk by chunk (ragged K, rows off 16 bytes); 0 = anything else (the two tiles built with the element-wise loader)."""
    es = a.element_size()
    if not (a.stride(1) == 1 and a.stride(0) >= a.shape[1]):
        return 0
    aligned = (a.stride(0) * es) % 16 == 0 and a.data_ptr() % 16 == 0 and b.data_ptr() % 16 == 0
    if b.stride(1) == 1 and b.stride(0) >= b.shape[1]:
        return 1 if aligned and (b.stride(0) * es) % 16 == 0 and b.shape[1] % (16 // es) == 0 else 3
    if b.stride(0) == 1 and b.stride(1) >= b.shape[0]:
        return 2 if aligned and (b.stride(1) * es) % 16 == 0 else 4
    return 0


def dma_operands(a, b):
    """``(a, b)`` as the direct-to-LDS loaders take them.  Operands of layout class 0 -- an A that is not row-major, a
    B that is neither row-major nor k-contiguous, rows that overlap -- would run on the chunk-wise loader at about
    a sixth of the speed (4096^3 bf16, column-major A: 242 against 1312 TFLOP/s); the wrappers below copy the
    offending operand into a row-major buffer first, which costs one pass over it.  The kernel objects themselves
    (``matmul_kernel[grid](...)``) take any strides as they are."""
    if dma_layout(a, b) != 0:
        return a, b
    if not (a.stride(1) == 1 and a.stride(0) >= a.shape[1]):
        a = a.contiguous()
    if not ((b.stride(1) == 1 and b.stride(0) >= b.shape[1]) or (b.stride(0) == 1 and b.stride(1) >= b.shape[0])):
        b = b.contiguous()
    return a, b


def _tuned_or_tune(op: str, key: tuple, kernel, launcher, fallback):
    """Config for ``key``: disk record, else a grid search (stored afterwards), else the built-in choice."""
    if not _autotune_enabled():
        return fallback()
    cfg = load_tuned(op, key)
    if cfg is not None:
        try:                      # a record written by another build may name a tile that no longer exists
            launcher(cfg)
            return cfg
        except (ValueError, RuntimeError):
            pass
    cfg = kernel.tune(launcher, **TUNE_OPTIONS)
    if cfg is None:
        raise RuntimeError(f"no HIP tile kernel accepts {op} {key}")
    save_tuned(op, key, cfg)
    return cfg


def run_memoised(memo: dict, op: str, key: tuple, kernel, launcher, fallback):
    """Launch with the config remembered for ``key`` (finding one first if there is none).

    A remembered config that the engine refuses for these very operands (``ValueError``: the layout changed in a
    way the key does not capture, or the memo was filled by hand) is replaced by the built-in choice for them.
    """
    if key not in memo:
        memo[key] = _tuned_or_tune(op, key, kernel, launcher, fallback)
    try:
        return launcher(memo[key])
    except ValueError:
        memo[key] = fallback()
        return launcher(memo[key])


def default_config(a, b, split=False):
    """The engine's built-in tile choice for this problem (used when tuning is switched off)."""
    import ctypes

    from tritonix_amd import _C
    from tritonix_amd.kernel import _torch_dtype_code

    g = _C.GemmArgs()
    g.m, g.k = a.shape
    g.n = b.shape[1]
    if a.dtype == torch.float32:
        # what the launch turns a float32 problem into: contiguous bf16 operands, three terms along K, fp32 result
        g.k = 3 * g.k
        g.stride_am, g.stride_ak, g.stride_bk, g.stride_bn = g.k, 1, g.n, 1
        g.in_dtype, g.out_dtype = _C.BF16, _C.F32
    else:
        g.stride_am, g.stride_ak = a.stride()
        g.stride_bk, g.stride_bn = b.stride()
        g.in_dtype = _torch_dtype_code(a.dtype)
        # base-pointer alignment decides between the two loaders; CPU tensors (host-side planning) count as aligned
        g.a = a.data_ptr() if a.is_cuda else None
        g.b = b.data_ptr() if b.is_cuda else None
    _C.load().tnx_gemm_default_config(ctypes.byref(g))
    cfg = {"block_m": g.block_m, "block_n": g.block_n, "block_k": g.block_k, "group_m": g.group_m,
           "num_stages": g.num_stages, "num_warps": g.num_warps}
    if split:
        cfg["split_k"] = max(2, g.split_k)
    elif g.split_k > 1:
        # shapes whose tiles alone leave CUs idle: the engine proposes a K cut for the plain kernel too
        cfg["split_k"] = g.split_k
    if g.tail_tiles > 0:
        cfg["tail_tiles"] = g.tail_tiles
    if g.schedule & _C.SCHED_SUPERBLOCK:
        cfg["superblock"] = 1
    if g.schedule & _C.SCHED_PERSISTENT:
        cfg["persistent"] = 1
    return cfg


def _autotune_enabled() -> bool:
    return os.environ.get("TRITONIX_AUTOTUNE", "1") not in ("0", "false", "False")


def _compute_units(device) -> int:
    """Workgroups of the large tiles that run together: the CU count of the device."""
    try:
        return int(torch.cuda.get_device_properties(device).multi_processor_count)
    except (RuntimeError, AssertionError):
        return 256


def _tile_or_split(a, b, key):
    """Config of ``triton_matmul`` for ``key``: the tuned tile, or -- for a problem whose output tiles alone leave
    CUs idle (fewer 64x128 tiles than the device has CUs) -- whichever of the tuned tile and the tuned K split is
    faster on these very operands.  Both are configs of the same engine, so the variant a shape ends up on lives
    in the config memo (and in the tuned-config record on disk), not in the dispatcher: its winner names stay the
    reference's two, ``"triton"`` and ``"pytorch"`` (tritonix/ops/matmul.py:291-293)."""
    from tritonix_amd.testing import do_bench

    tile = _tuned_or_tune("matmul", key, matmul_kernel, lambda cfg: _launch_matmul(a, b, cfg), lambda: default_config(a, b))
    m, n = a.shape[0], b.shape[1]
    if not _autotune_enabled() or "split_k" in tile or cdiv(m, 64) * cdiv(n, 128) >= _compute_units(a.device):
        return tile
    try:
        cut = _tuned_or_tune("matmul_cut", key, gemm_splitk_kernel, lambda cfg: _launch_splitk(a, b, cfg),
                             lambda: default_config(a, b, split=True))
        t_tile = do_bench(lambda: _launch_matmul(a, b, tile), **TUNE_OPTIONS)
        t_cut = do_bench(lambda: _launch_matmul(a, b, cut), **TUNE_OPTIONS)
    except (ValueError, RuntimeError):
        return tile
    if t_cut < t_tile:
        save_tuned("matmul", key, cut)
        return cut
    return tile


def triton_matmul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """C = A @ B on the HIP tile kernel, tile config tuned once per (m, n, k, dtype, layout class).

    Keeps the reference's name: callers and the ``"triton"`` backend label of
    ``matmul`` refer to it.  ``hip_matmul`` is the same function.  For thin problems the tuned config may carry a
    K split (``_tile_or_split``).
    """
    _check_2d(a, b)
    a, b = dma_operands(a, b)
    m, k = a.shape
    _, n = b.shape
    key = (m, n, k, a.dtype, dma_layout(a, b))
    if key not in _matmul_cfg:
        _matmul_cfg[key] = _tile_or_split(a, b, key)
    return run_memoised(_matmul_cfg, "matmul", key, matmul_kernel, lambda cfg: _launch_matmul(a, b, cfg),
                        lambda: default_config(a, b))


hip_matmul = triton_matmul


def matmul_splitk(a: torch.Tensor, b: torch.Tensor, split_k: int = 4) -> torch.Tensor:
    """Split-K GEMM for skinny shapes.

    As in the reference (tritonix/ops/matmul.py:280-288) ``split_k`` only keys
    the config memo; the split factor launched is the one the tuner picked.
    """
    _check_2d(a, b)
    a, b = dma_operands(a, b)
    m, k = a.shape
    _, n = b.shape
    key = (m, n, k, split_k, a.dtype, dma_layout(a, b))
    return run_memoised(_splitk_cfg, "matmul_splitk", key, gemm_splitk_kernel, lambda cfg: _launch_splitk(a, b, cfg),
                        lambda: default_config(a, b, split=True))


# the m <= 16 kernel: eight waves of a workgroup each take an eighth of K and meet in LDS
SKINNY_CONFIG = {"block_m": 16, "block_n": 32, "block_k": 32, "group_m": 8, "split_k": 8, "num_stages": 4,
                 "num_warps": 8}


def matmul_skinny(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """C = A @ B for at most 16 rows on the wavefront-level split-K kernel; ``ValueError`` for any other shape.

    Callable on its own; neither ``matmul`` nor ``triton_matmul`` selects it: a workgroup that keeps all of K to
    itself can own 32 columns at most before the 256 CUs run out of workgroups, and 64-byte row segments stream
    B at a quarter of what the cross-workgroup hand-over of the tile kernel reaches on the same shape."""
    _check_2d(a, b)
    return _launch_splitk(a, b, SKINNY_CONFIG)


# ``matmul`` keeps the reference's two backends and their names (tritonix/ops/matmul.py:291-293): "triton" is the
# HIP tile engine (its tile / K-split choice is made inside ``triton_matmul``), "pytorch" is ``torch.matmul``.
# The race times "triton" only: ``torch.matmul`` is the correctness oracle, reached with
# ``force_backend("pytorch")`` and never chosen, so an unforced ``matmul(a, b)`` always runs a kernel of this
# library and ``cache`` / ``timings`` hold no other name than the reference's.
matmul = dynamic_dispatch({"triton": triton_matmul}, key=["a", "b"])
matmul.register("pytorch", torch.matmul, raced=False)
matmul.alias("hip", "triton")
