"""The grid tuner over the real tile spaces, with the C library deciding what can launch (no GPU).

The launcher binds each config exactly as a launch would (HipKernel.make_args) and asks ``tnx_gemm_supported``;
its status becomes the exception a real launch raises (OutOfResources for the 160 KiB LDS budget, ValueError
for a tile that is not built), which is what the tuner prunes and skips on (tritonix/autotune.py:130-138 of the
reference).  Times come from a formula, so the outcome is known in advance.
"""
import ctypes

import pytest
import torch

import tritonix_amd
from tritonix_amd import _C
from tritonix_amd.testing import OutOfResources


class LibraryHarness:
    def __init__(self, kernel, a, b, c, formula, **extra):
        self.kernel, self.a, self.b, self.c, self.formula, self.extra = kernel, a, b, c, formula, extra
        self.timed, self.oom, self.skipped, self.current = [], [], [], None

    def launcher(self, cfg):
        self.current = cfg
        m, k = self.a.shape
        n = self.b.shape[1]
        bound = self.kernel._bind((self.a, self.b, self.c, m, n, k, self.a.stride(0), self.a.stride(1), self.b.stride(0),
                                   self.b.stride(1), self.c.stride(0), self.c.stride(1)), dict(cfg, **self.extra))
        g = self.kernel.make_args(bound)
        status = _C.load().tnx_gemm_supported(ctypes.byref(g))
        try:
            _C.raise_for_status(status, g)
        except OutOfResources:
            self.oom.append(dict(cfg))
            raise
        except ValueError:
            self.skipped.append(dict(cfg))
            raise
        self.timed.append(dict(cfg))

    def timer(self, fn, warmup=None, rep=None):
        fn()
        return self.formula(self.current)


def lds(cfg, es):
    return cfg["num_stages"] * (cfg["block_m"] * cfg["block_k"] + cfg["block_k"] * cfg["block_n"]) * es


def big_tiles_win(cfg):
    return 1e6 / (cfg["block_m"] * cfg["block_n"]) + 1.0 / cfg["block_k"] + 0.01 * cfg["num_stages"] + 0.001 * cfg["num_warps"]


@pytest.mark.parametrize("dtype,es", [(torch.bfloat16, 2), (torch.int8, 1)])
def test_matmul_space_against_the_library(dtype, es):
    a, b = torch.zeros(1024, 1024, dtype=dtype), torch.zeros(1024, 1024, dtype=dtype)
    c = torch.zeros(1024, 1024, dtype=torch.int32 if dtype == torch.int8 else dtype)
    kernel = tritonix_amd.matmul_kernel
    h = LibraryHarness(kernel, a, b, c, big_tiles_win)
    best = kernel.tune(h.launcher, bench_fn=h.timer)
    space = kernel.configs()
    assert len(space) == 3 * 3 * 3 * 2 * 3 * 2
    # everything that was timed fits the LDS budget and names a built kernel; the best of them comes back
    assert h.timed and all(lds(cfg, es) <= 163840 for cfg in h.timed)
    assert best == min(h.timed, key=big_tiles_win)
    assert (best["block_m"], best["block_n"]) == (256, 256)
    # every failed launch really was over budget, and nothing at or above a failed config (in the memory
    # parameters) was launched afterwards
    assert h.oom and all(lds(cfg, es) > 163840 for cfg in h.oom)
    mem = ("block_m", "block_n", "block_k", "num_stages")
    for bad in h.oom:
        later = h.timed[:]                                  # order inside `timed` does not matter for the claim below
        assert not any(all(cfg[p] >= bad[p] for p in mem) for cfg in later)
    # configs without a kernel (e.g. int8 with a 32-byte K slab) are skipped one by one, not pruned
    assert all(lds(cfg, es) <= 163840 for cfg in h.skipped)
    tried = len(h.timed) + len(h.oom) + len(h.skipped)
    assert tried <= len(space)
    # the pruners did their job: far fewer launches than the space has points
    assert len(h.oom) < sum(1 for cfg in space if lds(cfg, es) > 163840)


def test_splitk_space_prefers_enough_workgroups():
    a, b = torch.zeros(16, 14336, dtype=torch.bfloat16), torch.zeros(14336, 4096, dtype=torch.bfloat16)
    c = torch.zeros(16, 4096, dtype=torch.bfloat16)
    kernel = tritonix_amd.gemm_splitk_kernel

    def streaming(cfg):        # time falls with the number of workgroups up to 256, then rises with the slice count
        wgs = (4096 // cfg["block_n"]) * cfg["split_k"]
        return 1000.0 / min(wgs, 256) + 0.05 * cfg["split_k"] + 0.001 * cfg["block_m"] + 0.0001 * cfg["num_stages"]

    h = LibraryHarness(kernel, a, b, c, streaming)
    best = kernel.tune(h.launcher, bench_fn=h.timer)
    assert best == min(h.timed, key=streaming)
    assert (4096 // best["block_n"]) * best["split_k"] >= 256
    assert all(cfg["block_m"] >= 16 for cfg in h.timed)
    # the m <= 16 wave-split kernel is in the space too (16 x 32 x 32, eight waves, eight slices)
    assert any(cfg["block_m"] == 16 and cfg["block_n"] == 32 for cfg in h.timed) or \
        any(cfg["block_m"] == 16 and cfg["block_n"] == 32 for cfg in h.skipped)


def test_glu_space_rejects_int8():
    a, b = torch.zeros(256, 256, dtype=torch.int8), torch.zeros(256, 512, dtype=torch.int8)
    z = torch.zeros(256, 256, dtype=torch.int32)
    kernel = tritonix_amd.glu_kernel
    h = LibraryHarness(kernel, a, b, z, big_tiles_win, activation="silu")
    assert kernel.tune(h.launcher, bench_fn=h.timer, max_configs=5) is None      # nothing can launch: tune() says so
    assert not h.timed
