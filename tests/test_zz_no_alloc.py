"""tnx_gemm_static_workspace (the entry point that allocates nothing) against tnx_gemm, through the C ABI.

Two calls in a row on one GPU, the second with a smaller problem: the static scratch keeps the first call's
contents, so the second call only passes if what must start at zero is cleared and nothing stale is read."""
import ctypes

import pytest
import torch

import oracle
from tritonix_amd import _C

pytestmark = pytest.mark.gpu


def fill(a, b, c, split_k, tile, tail=0, schedule=0):
    g = _C.GemmArgs()
    g.a, g.b, g.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
    g.m, g.k = a.shape
    g.n = b.shape[1]
    g.stride_am, g.stride_ak = a.stride()
    g.stride_bk, g.stride_bn = b.stride()
    g.stride_cm, g.stride_cn = c.stride()
    code = {torch.bfloat16: _C.BF16, torch.float16: _C.F16, torch.int8: _C.I8, torch.int32: _C.I32}
    g.in_dtype, g.out_dtype = code[a.dtype], code[c.dtype]
    g.block_m, g.block_n, g.block_k, g.num_warps, g.num_stages = tile
    g.group_m, g.split_k, g.tail_tiles, g.epilogue = 8, split_k, tail, _C.EPI_NONE
    g.schedule = schedule
    g.stream = torch.cuda.current_stream().cuda_stream
    return g


def both_ways(lib, a, b, split_k, tile, tail=0):
    out_dt = torch.int32 if a.dtype == torch.int8 else a.dtype
    c_ws = torch.full((a.shape[0], b.shape[1]), 7, device=a.device, dtype=out_dt)
    c_static = torch.full_like(c_ws, 9)
    g = fill(a, b, c_ws, split_k, tile, tail)
    need = lib.tnx_gemm_workspace_bytes(ctypes.byref(g))
    ws = torch.zeros(max(need, 256), dtype=torch.uint8, device=a.device)
    g.workspace, g.workspace_bytes = ws.data_ptr(), ws.numel()
    assert lib.tnx_gemm(ctypes.byref(g)) == _C.OK
    h = fill(a, b, c_static, split_k, tile, tail)           # no workspace passed at all
    before = torch.cuda.memory_allocated()
    assert lib.tnx_gemm_static_workspace(ctypes.byref(h)) == _C.OK
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return c_ws, c_static, need


def test_static_workspace_matches_tnx_gemm_on_two_calls_in_a_row(device):
    lib = _C.load()
    # first call: the full skinny benchmark shape, K cut 8 ways (8.06 MiB of scratch)
    a, b = oracle.make_inputs("C3")
    c_ws, c_static, need = both_ways(lib, a.to(device), b.to(device), 8, (64, 128, 64, 8, 3))
    assert 0 < need <= _C.STATIC_WORKSPACE_BYTES
    assert torch.equal(c_ws, c_static)                        # same kernels, same order of summation: bit for bit
    assert oracle.within_tolerance(c_static, oracle.reference_matmul(a, b))[0]
    # second call, smaller: fewer tiles, fewer slices, another tile shape; stale slices and counters must not matter
    a2, b2 = oracle.make_inputs("C3", scale_down=4)
    c_ws2, c_static2, need2 = both_ways(lib, a2.to(device), b2.to(device), 4, (64, 128, 64, 4, 3))
    assert 0 < need2 < need
    assert torch.equal(c_ws2, c_static2)
    assert oracle.within_tolerance(c_static2, oracle.reference_matmul(a2, b2))[0]
    # third: int8, only the trailing tiles cut, exact
    a3, b3 = oracle.make_inputs("C5", scale_down=8)
    c_ws3, c_static3, _ = both_ways(lib, a3.to(device), b3.to(device), 2, (128, 128, 128, 4, 2), tail=8)
    assert torch.equal(c_ws3, c_static3) and torch.equal(c_static3.cpu(), oracle.reference_matmul(a3, b3))


def test_static_workspace_without_a_split_and_beyond_its_limit(device):
    lib = _C.load()
    a, b = oracle.make_inputs("C1")
    ad, bd = a.to(device), b.to(device)
    c = torch.empty((1024, 768), device=device, dtype=torch.float16)
    g = fill(ad, bd, c, 1, (128, 128, 64, 4, 2))
    assert lib.tnx_gemm_static_workspace(ctypes.byref(g)) == _C.OK       # no scratch needed: plain launch
    torch.cuda.synchronize()
    assert oracle.within_tolerance(c, oracle.reference_matmul(a, b))[0]
    # 16 slices of 48 tiles of 128x128 fp32 = 48 MiB > the static 32 MiB: refused with its own status, C untouched
    c.fill_(3)
    g = fill(ad, bd, c, 16, (128, 128, 64, 4, 2))
    assert lib.tnx_gemm_workspace_bytes(ctypes.byref(g)) > _C.STATIC_WORKSPACE_BYTES
    assert lib.tnx_gemm_static_workspace(ctypes.byref(g)) == _C.E_STATIC_LIMIT
    torch.cuda.synchronize()
    assert float(c.float().min()) == 3.0 == float(c.float().max())
    assert b"TNX_STATIC_WORKSPACE_BYTES" in lib.tnx_strerror(_C.E_STATIC_LIMIT)


def test_atomic_reduction_after_an_ordered_call_on_the_static_buffer(device):
    """The atomic reduction adds every K slice into one copy behind the counters and needs that copy zero at launch;
    an ordered call leaves its slices exactly there.  The entry point clears what the atomic launch will add into,
    so the order of the two calls does not matter: int8, exact against the oracle, twice in each order."""
    lib = _C.load()
    a, b = oracle.make_inputs("C5", scale_down=8)                      # 1024^3 int8
    ad, bd = a.to(device), b.to(device)
    ref = oracle.reference_matmul(a, b)
    tile = (128, 128, 128, 4, 2)
    for schedules in ((0, _C.SCHED_ATOMIC_REDUCE), (_C.SCHED_ATOMIC_REDUCE, 0), (_C.SCHED_ATOMIC_REDUCE, _C.SCHED_ATOMIC_REDUCE)):
        for schedule in schedules:
            c = torch.full((1024, 1024), -5, device=device, dtype=torch.int32)
            g = fill(ad, bd, c, 4, tile, schedule=schedule)
            before = torch.cuda.memory_allocated()
            assert lib.tnx_gemm_static_workspace(ctypes.byref(g)) == _C.OK
            assert torch.cuda.memory_allocated() == before
            torch.cuda.synchronize()
            assert torch.equal(c.cpu(), ref), f"schedule {schedule} after {schedules}"
    # a float problem of another tile shape after them: the atomic sums are order-dependent in the last bits only
    a2, b2 = oracle.make_inputs("C3", scale_down=4)
    c2 = torch.empty((a2.shape[0], b2.shape[1]), device=device, dtype=torch.bfloat16)
    g = fill(a2.to(device), b2.to(device), c2, 4, (64, 128, 64, 8, 3), schedule=_C.SCHED_ATOMIC_REDUCE)
    assert lib.tnx_gemm_static_workspace(ctypes.byref(g)) == _C.OK
    torch.cuda.synchronize()
    assert oracle.within_tolerance(c2, oracle.reference_matmul(a2, b2))[0]
