"""The launches inside a captured HIP graph: the library allocates nothing, clears nothing with a memset and keeps no
state but the split-K counters, which every launch leaves at zero, so a serving loop can capture a sequence of calls
once and replay it.  The graph is replayed several times with new operand contents, eager launches and
synchronisations between the replays, and every replay is compared bit for bit with the eager result."""
import pytest
import torch

import oracle
import tritonix_amd
from tritonix_amd.ops import matmul as mm
from tritonix_amd.ops.conv2d import conv2d_forward

pytestmark = pytest.mark.gpu


def test_a_captured_sequence_replays_with_the_eager_bits(device, monkeypatch):
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")          # the built-in tiles: no timing runs inside the capture
    g = torch.Generator().manual_seed(11)

    def draw(*shape, dtype=torch.bfloat16, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(dtype).to(device)

    a, b = draw(1024, 512, dtype=torch.float16), draw(512, 768, dtype=torch.float16, scale=0.05)     # one tile wave, uncut
    xs, ws = draw(16, 4096), draw(4096, 2048, scale=0.02)                                             # skinny: K cut, counters
    xg, w12 = draw(512, 1024), draw(1024, 2048, scale=0.03)                                           # gated epilogue
    ai = torch.randint(-127, 128, (256, 512), generator=g, dtype=torch.int8).to(device)
    bi = torch.randint(-127, 128, (512, 384), generator=g, dtype=torch.int8).to(device)
    img, w1, w3, bias = draw(4, 64, 14, 14), draw(128, 64, 1, 1, scale=0.1), draw(64, 64, 3, 3, scale=0.05), draw(128)
    inputs = [a, b, xs, ws, xg, w12, img, w1, w3, bias]

    def step():
        h = tritonix_amd.triton_matmul(a, b)
        return [h, tritonix_amd.triton_matmul(h, b.t()),            # a launch fed by a launch; k-contiguous B
                tritonix_amd.matmul_splitk(xs, ws), tritonix_amd.swiglu(xg, w12), tritonix_amd.triton_matmul(ai, bi),
                conv2d_forward(img, w1, bias),                      # TRITONIX_AUTOTUNE=0: the library's choice, untimed
                conv2d_forward(img, w3, None, (1, 1), (1, 1), (1, 1),
                               config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64)),
                conv2d_forward(img, w3, None, (2, 2), (1, 1), (1, 1),
                               config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64))]

    first = step()
    assert oracle.within_tolerance(first[0], oracle.reference_matmul(a, b))[0]
    assert oracle.within_tolerance(first[2], oracle.reference_matmul(xs, ws))[0]
    assert torch.equal(first[4].cpu(), oracle.reference_matmul(ai, bi))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):          # the split-K workspace of this stream and every memoised tile exist before the capture
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        outs = step()
    torch.cuda.synchronize()

    for replay in range(4):
        for t in inputs:            # new contents in the captured tensors
            t.copy_((torch.randn(t.shape, generator=g) * float(t.float().std().cpu())).to(t.dtype))
        want = [o.clone() for o in step()]          # eager launches between the replays
        torch.cuda.synchronize()
        for o in outs:
            o.fill_(7)
        graph.replay()
        torch.cuda.synchronize()
        for i, (o, w) in enumerate(zip(outs, want)):
            assert torch.equal(o, w), (replay, i)
    assert oracle.within_tolerance(outs[2], oracle.reference_matmul(xs, ws))[0]
    assert oracle.within_tolerance(outs[5], oracle.reference_conv2d(img, w1, bias))[0]
