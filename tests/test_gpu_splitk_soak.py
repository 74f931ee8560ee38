"""Split-K hand-over under repetition: many back-to-back launches over mixed shapes, split factors and trailing-tile
cuts, two workspaces used alternately, every result compared bit for bit with the first result of its case (the
slices are summed in slice order, so the result may not depend on which workgroup arrives last) and that first
result checked against the CPU oracle.  A stale read of a slice or of a counter would show as a mismatch."""
import ctypes

import pytest
import torch

import oracle
from tritonix_amd import _C

pytestmark = pytest.mark.gpu

CODE = {torch.bfloat16: _C.BF16, torch.float16: _C.F16, torch.int8: _C.I8, torch.int32: _C.I32}

# (dtype, m, n, k, (bm, bn, bk, warps, stages), split_k, tail_tiles)
CASES = [
    (torch.bfloat16, 16, 2048, 7168, (64, 128, 64, 8, 3), 8, 0),
    (torch.bfloat16, 16, 4096, 3584, (64, 128, 64, 4, 3), 4, 0),
    (torch.bfloat16, 48, 1024, 4096, (64, 128, 64, 8, 3), 16, 0),
    (torch.float16, 512, 2048, 2048, (128, 128, 64, 4, 3), 2, 0),
    (torch.float16, 1280, 1280, 1024, (128, 128, 64, 4, 3), 4, 36),      # 100 tiles, the last 36 cut
    (torch.bfloat16, 1536, 1536, 2048, (256, 256, 64, 4, 2), 4, 4),       # 36 tiles, the last 4 cut
    (torch.bfloat16, 100, 264, 2048, (128, 128, 64, 4, 2), 3, 0),         # ragged M and N, split not a power of two
    (torch.int8, 64, 2048, 8192, (64, 128, 128, 4, 3), 8, 0),
    (torch.int8, 1024, 1024, 2048, (128, 128, 128, 4, 2), 2, 16),
    (torch.bfloat16, 16, 512, 512, (64, 128, 64, 4, 3), 16, 0),           # more slices than K slabs
]


def inputs(dtype, m, n, k, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    if dtype == torch.int8:
        return (torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8),
                torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8))
    return torch.randn(m, k, generator=g).to(dtype), (torch.randn(k, n, generator=g) / k ** 0.5).to(dtype)


def test_back_to_back_splitk_launches_are_bit_stable(device):
    lib = _C.load()
    stream = torch.cuda.current_stream().cuda_stream
    prepared, biggest = [], 0
    for idx, (dtype, m, n, k, tile, split_k, tail) in enumerate(CASES):
        a, b = inputs(dtype, m, n, k, 100 + idx)
        ad, bd = a.to(device), b.to(device)
        out_dt = torch.int32 if dtype == torch.int8 else dtype
        outs = [torch.empty((m, n), device=device, dtype=out_dt) for _ in range(2)]
        args = []
        for c in outs:
            g = _C.GemmArgs()
            g.a, g.b, g.c = ad.data_ptr(), bd.data_ptr(), c.data_ptr()
            g.m, g.n, g.k = m, n, k
            g.stride_am, g.stride_ak, g.stride_bk, g.stride_bn, g.stride_cm, g.stride_cn = k, 1, n, 1, n, 1
            g.in_dtype, g.out_dtype = CODE[dtype], CODE[out_dt]
            g.block_m, g.block_n, g.block_k, g.num_warps, g.num_stages = tile
            g.group_m, g.split_k, g.tail_tiles, g.epilogue, g.stream = 8, split_k, tail, _C.EPI_NONE, stream
            args.append(g)
        biggest = max(biggest, lib.tnx_gemm_workspace_bytes(ctypes.byref(args[0])))
        prepared.append(dict(a=a, b=b, keep=(ad, bd), outs=outs, args=args, first=None))
    workspaces = [torch.zeros(biggest, dtype=torch.uint8, device=device) for _ in range(2)]

    launches = 0
    for rnd in range(27):                                       # 27 rounds x 10 cases x 2 outputs = 540 launches
        for idx, case in enumerate(prepared):
            for slot in range(2):
                g = case["args"][slot]
                ws = workspaces[(launches + rnd) % 2]
                g.workspace, g.workspace_bytes = ws.data_ptr(), ws.numel()
                assert lib.tnx_gemm(ctypes.byref(g)) == _C.OK, (rnd, idx)
                launches += 1
        torch.cuda.synchronize()
        for idx, case in enumerate(prepared):
            if case["first"] is None:
                first = case["outs"][0].clone()
                ref = oracle.reference_matmul(case["a"], case["b"])
                if first.dtype == torch.int32:
                    assert torch.equal(first.cpu(), ref), f"case {idx} differs from the oracle"
                else:
                    assert oracle.within_tolerance(first, ref)[0], f"case {idx} outside tolerance"
                case["first"] = first
            for slot in range(2):
                assert torch.equal(case["outs"][slot], case["first"]), f"round {rnd} case {idx} output {slot}: result changed"
                case["outs"][slot].fill_(1)                    # a launch that writes nothing must not pass on old data
    assert launches >= 500
    # every launch left its arrival counters at zero in both workspaces
    for ws in workspaces:
        assert int(ws[:65536].view(torch.int32).abs().max()) == 0
