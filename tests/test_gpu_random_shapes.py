"""Seeded random problems through every built tile: shapes from 1 to about a thousand in each dimension (ragged
against every tile size), both operand layouts the DMA loaders take, base pointers and row pitches at odd
element offsets, K cut with and without a tail-only cut, the super-block order, the gated epilogue.  The operands
are views into buffers filled with NaN (int8: 77), so a value taken from outside a matrix shows.  int8 results are
compared exactly, float results within the tolerance of the parity tests."""
import importlib
import random

import pytest
import torch

from tritonix_amd import _C

mm = importlib.import_module("tritonix_amd.ops.matmul")
sg = importlib.import_module("tritonix_amd.ops.swiglu")

pytestmark = pytest.mark.gpu
DTYPES = {"bf16": torch.bfloat16, "f16": torch.float16, "i8": torch.int8}


def embedded(mat, offset, pad, fill, device):
    """`mat` as a view with row pitch cols + pad, `offset` elements into a buffer of `fill`."""
    rows, cols = mat.shape
    buf = torch.full((rows * (cols + pad) + 64,), fill, dtype=mat.dtype)
    buf[offset:offset + rows * (cols + pad)].view(rows, cols + pad)[:, :cols] = mat
    return buf.to(device)[offset:offset + rows * (cols + pad)].view(rows, cols + pad)[:, :cols]


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_problems_on_random_tiles(device, seed):
    rnd = random.Random(seed)
    tiles = {"bf16": [], "f16": [], "i8": []}
    for name in _C.kernel_names():
        f = name.split()
        tiles[f[0]].append(tuple(int(v) for v in f[1:6]) + ("bt" in f[6:],))
    ran = 0
    for case in range(120):
        dt = rnd.choice(["bf16", "bf16", "f16", "i8"])
        bm, bn, bk, nw, st, has_bt = rnd.choice(tiles[dt])
        m = rnd.choice([1, 5, 16, 63, 64, 100, 257, 300, 513, 1025])
        n = rnd.choice([1, 8, 24, 100, 129, 256, 264, 517, 1000, 2050])
        k = rnd.choice([1, 7, 40, 64, 65, 128, 200, 517, 1024, 1031, 2056])
        layout = rnd.choice(["row-major", "row-major", "k-contiguous"]) if has_bt else "row-major"
        glu = dt != "i8" and rnd.random() < 0.2 and n % 2 == 0 and layout == "row-major"
        split = 1 if glu else rnd.choice([1, 1, 1, 2, 4])
        off_a, off_b = rnd.choice([0, 0, 1, 3, 8]), rnd.choice([0, 0, 1, 5, 8])
        pad_a, pad_b = rnd.choice([0, 0, 1, 8]), rnd.choice([0, 0, 3, 8])
        dtype = DTYPES[dt]
        g = torch.Generator("cpu").manual_seed(1000 * seed + case)
        if dt == "i8":
            a = torch.randint(-127, 128, (m, k), generator=g, dtype=dtype)
            b = torch.randint(-127, 128, (k, n), generator=g, dtype=dtype)
            fill = 77
        else:
            a = torch.randn(m, k, generator=g).to(dtype)
            b = (torch.randn(k, n, generator=g) / k ** 0.5).to(dtype)
            fill = float("nan")
        ad = embedded(a, off_a, pad_a, fill, device)
        bd = embedded(b, off_b, pad_b, fill, device) if layout == "row-major" else \
            embedded(b.t().contiguous(), off_b, pad_b, fill, device).t()
        cfg = dict(block_m=bm, block_n=bn, block_k=bk, group_m=rnd.choice([1, 4, 8]), num_stages=st, num_warps=nw)
        if split > 1:
            cfg["split_k"] = split
            if rnd.random() < 0.4:
                cfg["tail_tiles"] = rnd.choice([1, 2, 3, 7])
        elif rnd.random() < 0.3:
            cfg["superblock"] = 1
        what = f"seed {seed} case {case}: {dt} {m}x{n}x{k} B {layout}, {cfg}, glu {glu}, offsets {off_a},{off_b}, pads {pad_a},{pad_b}"
        if glu:
            out = sg._launch_glu(ad, bd, cfg, "silu")
        elif split > 1:
            out = mm._launch_splitk(ad, bd, cfg)
        else:
            out = mm._launch_matmul(ad, bd, cfg)
        torch.cuda.synchronize()
        ran += 1
        if dt == "i8":
            assert torch.equal(out.cpu(), (a.double() @ b.double()).to(torch.int32)), what
            continue
        y = a.float() @ b.float()
        ref = torch.nn.functional.silu(y[:, 0::2]) * y[:, 1::2] if glu else y
        got = out.cpu().float()
        assert bool(torch.isfinite(got).all()), what
        bound = 1e-2 * ref.abs() + 1e-2 * ref.pow(2).mean().sqrt() + 1e-3
        assert bool(((got - ref).abs() <= bound).all()), what
    assert ran == 120


@pytest.mark.parametrize("seed", [0, 1])
def test_random_float32_problems(device, seed):
    """float32 operands (a three-term bf16 split inside the launch) on every tile that carries the fp32 epilogue:
    NaN-embedded strided views, both layouts, K cuts and the gated epilogue; error bound 2e-4 of the largest result
    against the float64 product, fifty times tighter than the 16-bit bar."""
    rnd = random.Random(100 + seed)
    tiles = []
    for name in _C.kernel_names():
        f = name.split()
        if f[0] == "bf16" and int(f[1]) * int(f[2]) <= 128 * 128:
            tiles.append(tuple(int(v) for v in f[1:6]) + ("bt" in f[6:],))
    assert tiles
    for case in range(60):
        bm, bn, bk, nw, st, _ = rnd.choice(tiles)
        m = rnd.choice([1, 5, 16, 64, 100, 257, 513])
        n = rnd.choice([8, 24, 100, 256, 264, 1000])
        k = rnd.choice([1, 7, 40, 64, 200, 517, 1024])
        layout = rnd.choice(["row-major", "row-major", "k-contiguous", "column-major-a"])
        glu = rnd.random() < 0.2 and n % 2 == 0
        split = 1 if glu else rnd.choice([1, 1, 2, 4])
        g = torch.Generator("cpu").manual_seed(5000 * seed + case)
        a = torch.randn(m, k, generator=g)
        b = torch.randn(k, n, generator=g) / k ** 0.5
        fill = float("nan")
        ad = embedded(a, rnd.choice([0, 1, 3]), rnd.choice([0, 1, 8]), fill, device) if layout != "column-major-a" else \
            embedded(a.t().contiguous(), 1, 2, fill, device).t()
        bd = embedded(b, rnd.choice([0, 5]), rnd.choice([0, 3]), fill, device) if layout != "k-contiguous" else \
            embedded(b.t().contiguous(), 2, 1, fill, device).t()
        cfg = dict(block_m=bm, block_n=bn, block_k=bk, group_m=8, num_stages=st, num_warps=nw)
        if split > 1:
            cfg["split_k"] = split
        what = f"seed {seed} case {case}: f32 {m}x{n}x{k} {layout}, {cfg}, glu {glu}"
        if glu:
            out = sg._launch_glu(ad, bd, cfg, "silu")
        elif split > 1:
            out = mm._launch_splitk(ad, bd, cfg)
        else:
            out = mm._launch_matmul(ad, bd, cfg)
        torch.cuda.synchronize()
        assert out.dtype == torch.float32, what
        y = a.double() @ b.double()
        ref = torch.nn.functional.silu(y[:, 0::2]) * y[:, 1::2] if glu else y
        got = out.cpu().double()
        assert bool(torch.isfinite(got).all()), what
        assert float((got - ref).abs().max()) <= 2e-4 * max(float(ref.abs().max()), 1e-3) * (3 if glu else 1), what
