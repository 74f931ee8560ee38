"""conv2d forward on the GPU against the CPU oracle (tritonix/ops/conv2d/forward.py:19-165, :202-311).

Tolerance: the kernel accumulates in fp32 and rounds once to the 16-bit output type, the oracle keeps fp32; the
bar is the one of the GEMM tests, |out - ref| <= 1e-2 * (|ref| + rms(ref)).
"""
import numpy as np
import pytest
import torch

import oracle
from tritonix_amd import _C
from tritonix_amd.ops.conv2d import conv2d_forward, conv2d_forward_kernel, torch_conv2d_forward
from tritonix_amd.ops.conv2d import forward as conv

pytestmark = pytest.mark.gpu

CASES = {
    # n, c_in, h, w, c_out, r, s, stride, padding, dilation, bias
    "3x3_same": (2, 16, 16, 16, 32, 3, 3, (1, 1), (1, 1), (1, 1), True),
    "1x1_flat": (1, 8, 8, 8, 16, 1, 1, (1, 1), (0, 0), (1, 1), False),
    "7x7_stem_ragged_k": (3, 3, 19, 23, 20, 7, 7, (2, 2), (3, 3), (1, 1), True),
    "w_out_14": (2, 24, 14, 14, 40, 3, 3, (1, 1), (1, 1), (1, 1), True),
    "all_asymmetric": (2, 16, 17, 13, 24, 3, 2, (1, 2), (2, 0), (2, 1), False),
    "1x1_stride2": (2, 32, 28, 28, 64, 1, 1, (2, 2), (0, 0), (1, 1), False),
    "one_pixel": (1, 5, 5, 5, 7, 5, 5, (1, 1), (0, 0), (1, 1), True),
    "dilated_wide_pad": (2, 32, 9, 9, 200, 3, 3, (1, 1), (2, 2), (2, 2), True),
    "odd_plane_7x7": (3, 16, 7, 7, 24, 3, 3, (1, 1), (1, 1), (1, 1), True),
    "pad_wider_than_filter": (1, 8, 6, 6, 8, 3, 3, (1, 1), (4, 4), (1, 1), False),
    "tiny_tensor": (1, 1, 2, 3, 2, 1, 1, (1, 1), (0, 0), (1, 1), True),
}
TILES = [(64, 64, 32), (128, 128, 64), (64, 128, 64), (128, 64, 32), (256, 128, 64), (128, 256, 64)]   # BLOCK_SIZE_M, _N, _K


def _inputs(case, dtype, seed=0):
    n, c, h, w, k, r, s, stride, padding, dilation, has_bias = case
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, c, h, w, generator=g).to(dtype)
    wt = (torch.randn(k, c, r, s, generator=g) / (c * r * s) ** 0.5).to(dtype)
    b = torch.randn(k, generator=g).to(dtype) if has_bias else None
    return x, wt, b, stride, padding, dilation


def _oracle(x, wt, b, stride, padding, dilation):
    y = oracle.tiled_conv2d(x.float().numpy(), wt.float().numpy(), None if b is None else b.float().numpy(), stride, padding,
                            dilation, 32, 32, 16)
    return torch.from_numpy(y)


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_conv2d_matches_the_oracle(name, dtype, device):
    x, wt, b, stride, padding, dilation = _inputs(CASES[name], dtype, seed=len(name))
    ref = _oracle(x, wt, b, stride, padding, dilation)
    for bm, bn, bk in TILES:
        cfg = dict(BLOCK_SIZE_M=bm, BLOCK_SIZE_N=bn, BLOCK_SIZE_K=bk, GROUP_SIZE_M=4)
        out = conv2d_forward(x.to(device), wt.to(device), None if b is None else b.to(device), stride, padding, dilation,
                             config=cfg)
        assert out.dtype == dtype and tuple(out.shape) == tuple(ref.shape)
        ok, err, rel = oracle.within_tolerance(out, ref)
        assert ok, (name, dtype, cfg, err, rel)


# geometries the direct-to-LDS kernel accepts: stride_w == 1, c_in * R * S a multiple of 64
DMA_CASES = {
    "1x1": (2, 64, 16, 16, 128, 1, 1, (1, 1), (0, 0), (1, 1), False),
    "3x3_same": (2, 64, 16, 16, 128, 3, 3, (1, 1), (1, 1), (1, 1), True),
    "w_out_14_ragged_channels": (3, 64, 14, 14, 200, 3, 3, (1, 1), (1, 1), (1, 1), True),
    "w_out_7": (3, 128, 7, 7, 130, 3, 3, (1, 1), (1, 1), (1, 1), False),
    "stride_h_2_dilated": (2, 64, 17, 13, 96, 3, 3, (2, 1), (2, 2), (2, 2), True),
    "1x5_wide_pad": (2, 64, 9, 20, 64, 1, 5, (1, 1), (0, 3), (1, 1), True),
    "no_pad": (1, 192, 10, 10, 256, 3, 3, (1, 1), (0, 0), (1, 1), True),
    "5x5": (2, 64, 12, 12, 128, 5, 5, (1, 1), (2, 2), (1, 1), False),
    "w_out_3": (2, 64, 3, 3, 64, 3, 3, (1, 1), (1, 1), (1, 1), True),
    # 1x1, unit strides, no padding: the plane is handed to the kernel as one row (49 and 196 are not multiples of 8:
    # the last chunk of the tensor crosses its end)
    "1x1_plane_7x7": (3, 64, 7, 7, 130, 1, 1, (1, 1), (0, 0), (1, 1), True),
    "1x1_plane_14x14_dilated": (2, 128, 14, 14, 192, 1, 1, (1, 1), (0, 0), (2, 3), False),
}
DMA_TILES = [(128, 128, 64), (128, 256, 64), (256, 128, 64)]     # BLOCK_SIZE_M (pixels), BLOCK_SIZE_N (channels), BLOCK_SIZE_K


@pytest.mark.parametrize("name", sorted(DMA_CASES))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_direct_to_lds_loader_matches_the_oracle_and_the_register_kernel(name, dtype, device):
    """Padding rows come from the buffer bound, padding columns from the in-LDS fix-up, the first and last chunk of the
    tensor from the element-wise fill; every case has all three.  Both kernels add the same products in the same
    order (block_k = 64, the same MFMA shape), so they must agree bit for bit."""
    x, wt, b, stride, padding, dilation = _inputs(DMA_CASES[name], dtype, seed=len(name))
    ref = _oracle(x, wt, b, stride, padding, dilation)
    xd, wd, bd = x.to(device), wt.to(device), None if b is None else b.to(device)
    regs = conv2d_forward(xd, wd, bd, stride, padding, dilation,
                          config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, LOADER="registers"))
    for bm, bn, bk in DMA_TILES:
        cfg = dict(BLOCK_SIZE_M=bm, BLOCK_SIZE_N=bn, BLOCK_SIZE_K=bk, LOADER="dma")
        out = conv2d_forward(xd, wd, bd, stride, padding, dilation, config=cfg)
        ok, err, rel = oracle.within_tolerance(out, ref)
        assert ok, (name, dtype, cfg, err, rel)
        assert torch.equal(out, regs), (name, dtype, cfg)


def test_seeded_random_geometries_on_both_kernels(device):
    """Sixty geometries drawn from a fixed seed (filters 1-5 per side, dilation 1-3, padding 0-4, stride_h 1-3, planes
    3-40 wide, 64 or 128 input channels so that the direct-to-LDS kernel applies): the register-staged kernel against
    the CPU library routine in fp32, and the direct-to-LDS kernel bit for bit against the register-staged one."""
    rng = np.random.default_rng(2024)
    done = 0
    while done < 60:
        r, s_ = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        dil = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        pad = (int(rng.integers(0, 5)), int(rng.integers(0, 5)))
        stride = (int(rng.integers(1, 4)), 1)
        h, w = int(rng.integers(3, 41)), int(rng.integers(3, 41))
        c_in = int(rng.choice([64, 128]))
        c_out = int(rng.integers(1, 300))
        n = int(rng.integers(1, 4))
        ho, wo = conv.output_size(h, w, r, s_, stride, pad, dil)
        if ho <= 0 or wo <= 0 or (c_in * r * s_) % 64:
            continue
        done += 1
        g = torch.Generator().manual_seed(done)
        x = torch.randn(n, c_in, h, w, generator=g).bfloat16()
        wt = (torch.randn(c_out, c_in, r, s_, generator=g) / (c_in * r * s_) ** 0.5).bfloat16()
        b = torch.randn(c_out, generator=g).bfloat16() if done % 2 else None
        xd, wd, bd = x.to(device), wt.to(device), None if b is None else b.to(device)
        tile = [(128, 128), (128, 256), (256, 128)][done % 3]
        regs = conv2d_forward(xd, wd, bd, stride, pad, dil,
                              config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64, LOADER="registers"))
        dma = conv2d_forward(xd, wd, bd, stride, pad, dil,
                             config=dict(BLOCK_SIZE_M=tile[0], BLOCK_SIZE_N=tile[1], BLOCK_SIZE_K=64, LOADER="dma"))
        what = (done, n, c_in, h, w, c_out, r, s_, stride, pad, dil, tile)
        assert oracle.within_tolerance(regs, oracle.reference_conv2d(x, wt, b, stride, pad, dil))[0], what
        assert torch.equal(dma, regs), what


# 1x1 filters, unit stride, no padding: n, c_in, h, w, c_out, bias dtype (None: no bias)
GEMM_ROUTE_CASES = [
    (2, 64, 16, 16, 128, torch.float32),       # rows of 512 bytes, K one slab
    (3, 100, 13, 7, 70, "same"),               # ragged everywhere: c_in, plane of 91 pixels, channels
    (2, 256, 56, 56, 64, "same"),              # the large-image layer "auto" hands to this route
    (4, 2048, 7, 7, 512, None),                # long K, plane of 49 pixels (rows of 98 bytes)
    (33, 24, 5, 5, 40, "same"),                # many small images
    (1, 7, 3, 1, 5, torch.float32),            # smaller than one tile in every direction
    (2, 192, 14, 14, 1000, "same"),            # channels ragged against 64 and 128
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_route_for_1x1_layers(dtype, device):
    """A 1x1 layer is the GEMM out[n] = W x X[n] image by image; the GEMM route runs it on the GEMM tile kernels, all
    images in one grid, bias added to the fp32 sum.  Against the oracle on the library's own tile and on named tiles;
    with a 64-deep K slab it adds the same products in the same order as the conv2d kernels, so it must also agree
    with the register-staged kernel bit for bit."""
    for i, (n, c, h, w, k, bias) in enumerate(GEMM_ROUTE_CASES):
        g = torch.Generator().manual_seed(100 + i)
        x = torch.randn(n, c, h, w, generator=g).to(dtype)
        wt = (torch.randn(k, c, 1, 1, generator=g) / c ** 0.5).to(dtype)
        b = None if bias is None else torch.randn(k, generator=g).to(dtype if bias == "same" else bias)
        geo = ((1, 1), (0, 0), (1, 1))
        ref = oracle.reference_conv2d(x, wt, b, *geo)
        xd, wd, bd = x.to(device), wt.to(device), None if b is None else b.to(device)
        regs = conv2d_forward(xd, wd, bd, *geo, config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64, LOADER="registers"))
        assert oracle.within_tolerance(regs, ref)[0], (i, dtype)
        for (bm, bn, bk) in [(0, 0, 0), (64, 64, 64), (128, 128, 64), (128, 64, 64), (64, 32, 64), (128, 128, 32),
                             (64, 256, 64), (64, 256, 32)]:    # the last: wave tiles of 128 rows, two bias values per lane
            cfg = dict(BLOCK_SIZE_M=bm, BLOCK_SIZE_N=bn, BLOCK_SIZE_K=bk, LOADER="gemm")
            canvas = torch.full((n * k * h * w + 64,), float("nan"), dtype=dtype, device=device)
            out = canvas[32:32 + n * k * h * w].view(n, k, h, w)
            conv2d_forward_kernel[(1,)](out, xd, wd, bd, n, c, h, w, k, h, w, 1, 1, 1, 1, 0, 0, 1, 1, n * h * w, k, c,
                                        GROUP_SIZE_M=8, **cfg)
            ok, err, rel = oracle.within_tolerance(out, ref)
            assert ok, (i, dtype, cfg, err, rel)
            assert bool(torch.isnan(canvas[:32]).all()) and bool(torch.isnan(canvas[32 + n * k * h * w:]).all()), (i, dtype, cfg)
            if bk == 64 or bk == 0:
                assert torch.equal(out, regs), (i, dtype, cfg)


def test_seeded_random_1x1_layers_on_the_gemm_route(device):
    """Eighty 1x1 layers drawn from a fixed seed (1-40 images, 1-300 channels either side, planes 1-30 per side, bias of
    the tensor type, fp32 or none, the library's tile or one of the built ones): against the CPU library routine in
    fp32, the output embedded in NaN so that a store outside it shows."""
    rng = np.random.default_rng(77)
    gemm_tiles = sorted({(int(f[1]), int(f[2]), int(f[3])) for f in (x.split() for x in _C.kernel_names())
                         if f[0] == "bf16" and int(f[1]) * int(f[2]) <= 128 * 128})
    assert len(gemm_tiles) >= 8
    for case in range(80):
        n, c, k = int(rng.integers(1, 41)), int(rng.integers(1, 301)), int(rng.integers(1, 301))
        h, w = int(rng.integers(1, 31)), int(rng.integers(1, 31))
        dtype = [torch.bfloat16, torch.float16][case % 2]
        g = torch.Generator().manual_seed(1000 + case)
        x = torch.randn(n, c, h, w, generator=g).to(dtype)
        wt = (torch.randn(k, c, 1, 1, generator=g) / c ** 0.5).to(dtype)
        b = [None, torch.randn(k, generator=g).to(dtype), torch.randn(k, generator=g)][case % 3]
        bcout, bpix, bk = (0, 0, 0) if case % 4 == 0 else gemm_tiles[int(rng.integers(0, len(gemm_tiles)))]
        # every third case: output, input and weight start an odd number of elements into their allocations
        off = 25 if case % 3 == 1 else 24
        canvas = torch.full((n * k * h * w + 2 * off,), float("nan"), dtype=dtype, device=device)
        out = canvas[off:off + n * k * h * w].view(n, k, h, w)
        xd = torch.full((x.numel() + off,), float("nan"), dtype=dtype, device=device)
        xd[off:].copy_(x.reshape(-1))
        wd = torch.full((wt.numel() + off,), float("nan"), dtype=dtype, device=device)
        wd[off:].copy_(wt.reshape(-1))
        conv2d_forward_kernel[(1,)](out, xd[off:].view(n, c, h, w), wd[off:].view(k, c, 1, 1), None if b is None else b.to(device),
                                    n, c, h, w, k, h, w, 1, 1, 1, 1, 0, 0, 1, 1, n * h * w, k, c, BLOCK_SIZE_M=bpix,
                                    BLOCK_SIZE_N=bcout, BLOCK_SIZE_K=bk, GROUP_SIZE_M=8, LOADER="gemm")
        what = (case, n, c, h, w, k, dtype, None if b is None else b.dtype, bcout, bpix, bk, off)
        ok, err, rel = oracle.within_tolerance(out, oracle.reference_conv2d(x, wt, b))
        assert ok, (what, err, rel)
        assert bool(torch.isnan(canvas[:off]).all()) and bool(torch.isnan(canvas[off + n * k * h * w:]).all()), what


def test_gemm_route_follows_dilation_free_geometry_only(device):
    """Dilation has no effect on a single tap; stride or padding take the layer off the GEMM route."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 64, 12, 12, generator=g).bfloat16().to(device)
    wt = (torch.randn(96, 64, 1, 1, generator=g) / 8).bfloat16().to(device)
    cfg = dict(BLOCK_SIZE_M=0, BLOCK_SIZE_N=0, BLOCK_SIZE_K=0, LOADER="gemm")
    plain = conv2d_forward(x, wt, None, (1, 1), (0, 0), (1, 1), config=cfg)
    assert torch.equal(conv2d_forward(x, wt, None, (1, 1), (0, 0), (3, 2), config=cfg), plain)
    for stride, padding in (((2, 1), (0, 0)), ((1, 1), (0, 1))):
        with pytest.raises(ValueError):
            conv2d_forward(x, wt, None, stride, padding, (1, 1), config=cfg)


def test_tuner_times_the_gemm_route_on_1x1_layers(device):
    conv._CONV_FWD_CONFIG_CACHE.clear()
    g = torch.Generator().manual_seed(6)
    x = torch.randn(8, 256, 56, 56, generator=g).bfloat16()
    wt = (torch.randn(64, 256, 1, 1, generator=g) / 16).bfloat16()
    out = conv2d_forward(x.to(device), wt.to(device))
    assert oracle.within_tolerance(out[:1], oracle.reference_conv2d(x[:1], wt, None, (1, 1), (0, 0), (1, 1)))[0]
    (cfg,) = conv._CONV_FWD_CONFIG_CACHE.values()
    assert cfg.get("LOADER", "auto") in ("auto", "gemm")
    again = conv2d_forward(x.to(device), wt.to(device))
    assert torch.equal(out, again)


def test_loader_that_does_not_fit_is_refused(device):
    x, wt, b, stride, padding, dilation = _inputs(CASES["1x1_stride2"], torch.bfloat16)
    with pytest.raises(ValueError):           # stride_w == 2
        conv2d_forward(x.to(device), wt.to(device), None, stride, padding, dilation,
                       config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, LOADER="dma"))
    x, wt, b, stride, padding, dilation = _inputs(CASES["3x3_same"], torch.bfloat16)
    with pytest.raises(ValueError):           # c_in * 9 = 144 is not a multiple of 64
        conv2d_forward(x.to(device), wt.to(device), None, stride, padding, dilation,
                       config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, LOADER="dma"))
    # the same tile without the demand falls back to the register-staged kernel
    out = conv2d_forward(x.to(device), wt.to(device), None, stride, padding, dilation,
                         config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64))
    assert oracle.within_tolerance(out, _oracle(x, wt, None, stride, padding, dilation))[0]


def test_weight_that_is_not_16_byte_aligned_takes_the_register_kernel(device):
    x, wt, b, stride, padding, dilation = _inputs(DMA_CASES["3x3_same"], torch.bfloat16, seed=2)
    store = torch.empty(wt.numel() + 1, dtype=wt.dtype, device=device)
    wd = store[1:].view(wt.shape)                       # 2 bytes past a 16-byte boundary
    wd.copy_(wt)
    assert wd.data_ptr() % 16 == 2 and wd.is_contiguous()
    ref = _oracle(x, wt, b, stride, padding, dilation)
    cfg = dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64)
    out = conv2d_forward(x.to(device), wd, b.to(device), stride, padding, dilation, config=cfg)
    assert oracle.within_tolerance(out, ref)[0]
    with pytest.raises(ValueError):
        conv2d_forward(x.to(device), wd, b.to(device), stride, padding, dilation, config=dict(cfg, LOADER="dma"))
    # an input that is only 2-byte aligned is fine for both kernels
    xs = torch.empty(x.numel() + 1, dtype=x.dtype, device=device)
    xd = xs[1:].view(x.shape)
    xd.copy_(x)
    out = conv2d_forward(xd, wt.to(device), b.to(device), stride, padding, dilation, config=dict(cfg, LOADER="dma"))
    assert oracle.within_tolerance(out, ref)[0]
    # so is an output that is only 2-byte aligned (the epilogue's 16-byte stores take any element address)
    ys = torch.empty(ref.numel() + 1, dtype=x.dtype, device=device)
    yd = ys[1:].view(ref.shape)
    n, c, h, w = x.shape
    k, _, r, s_ = wt.shape
    conv2d_forward_kernel[(1,)](yd, xd, wt.to(device), b.to(device), n, c, h, w, k, ref.shape[2], ref.shape[3], r, s_, stride[0],
                                stride[1], padding[0], padding[1], dilation[0], dilation[1], n * ref.shape[2] * ref.shape[3], k,
                                c * r * s_, BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64, GROUP_SIZE_M=8, LOADER="dma")
    assert oracle.within_tolerance(yd, ref)[0]


def test_float32_bias_and_no_bias_agree_with_the_oracle(device):
    x, wt, _, stride, padding, dilation = _inputs(CASES["3x3_same"], torch.bfloat16, seed=3)
    b32 = torch.randn(wt.shape[0], generator=torch.Generator().manual_seed(4))
    out = conv2d_forward(x.to(device), wt.to(device), b32.to(device), stride, padding, dilation,
                         config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64))
    assert oracle.within_tolerance(out, _oracle(x, wt, b32, stride, padding, dilation))[0]


def test_tiles_agree_bit_for_bit_when_k_order_is_the_same(device):
    """Two tiles with the same block_k add the same products in the same order: their outputs are identical."""
    x, wt, b, stride, padding, dilation = _inputs(CASES["w_out_14"], torch.bfloat16, seed=7)
    outs = [conv2d_forward(x.to(device), wt.to(device), b.to(device), stride, padding, dilation,
                           config=dict(BLOCK_SIZE_M=bm, BLOCK_SIZE_N=bn, BLOCK_SIZE_K=64))
            for bm, bn in ((64, 64), (128, 128), (64, 128), (128, 64))]
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


def test_one_by_one_filter_equals_the_gemm_engine(device):
    """A 1x1, stride-1 conv is W[c_out, c_in] @ X[c_in, pixels] per image: the conv kernel and the GEMM kernel
    must round the same fp32 sums (same block_k, same accumulation order along k)."""
    import tritonix_amd

    g = torch.Generator().manual_seed(11)
    x = torch.randn(2, 64, 16, 16, generator=g).bfloat16().to(device)
    wt = (torch.randn(128, 64, 1, 1, generator=g) / 8).bfloat16().to(device)
    out = conv2d_forward(x, wt, None, config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64))
    for img in range(2):
        with tritonix_amd.matmul.force_backend("triton"):
            want = tritonix_amd.matmul(wt.view(128, 64), x[img].reshape(64, 256))
        assert oracle.within_tolerance(out[img].reshape(128, 256), want.float().cpu(), rel=4e-3)[0]


def test_mini_tuner_picks_a_candidate_and_remembers_it(device):
    conv._CONV_FWD_CONFIG_CACHE.clear()
    x, wt, b, stride, padding, dilation = _inputs(CASES["w_out_14"], torch.float16, seed=5)
    out = conv2d_forward(x.to(device), wt.to(device), b.to(device), stride, padding, dilation)
    assert len(conv._CONV_FWD_CONFIG_CACHE) == 1
    (key, cfg), = conv._CONV_FWD_CONFIG_CACHE.items()
    assert key[-1] == torch.float16 and set(cfg) == {"BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K", "GROUP_SIZE_M"}
    assert oracle.within_tolerance(out, _oracle(x, wt, b, stride, padding, dilation))[0]
    again = conv2d_forward(x.to(device), wt.to(device), b.to(device), stride, padding, dilation)
    assert torch.equal(out, again) and len(conv._CONV_FWD_CONFIG_CACHE) == 1


def test_kernel_launch_object_with_the_reference_arguments(device):
    x, wt, b, stride, padding, dilation = _inputs(CASES["all_asymmetric"], torch.bfloat16, seed=9)
    n, c, h, w = x.shape
    k, _, r, s = wt.shape
    ho, wo = conv.output_size(h, w, r, s, stride, padding, dilation)
    xd, wd = x.to(device), wt.to(device)
    out = torch.empty(n, k, ho, wo, dtype=x.dtype, device=device)
    grid = (conv.cdiv(n * ho * wo, 64), conv.cdiv(k, 64))
    conv2d_forward_kernel[grid](out, xd, wd, None, n, c, h, w, k, ho, wo, r, s, stride[0], stride[1], padding[0], padding[1],
                                dilation[0], dilation[1], n * ho * wo, k, c * r * s, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64,
                                BLOCK_SIZE_K=32, GROUP_SIZE_M=8, USE_TF32=True)
    assert oracle.within_tolerance(out, _oracle(x, wt, None, stride, padding, dilation))[0]


def test_through_the_c_abi_with_the_built_in_tile(device):
    import ctypes

    x, wt, b, stride, padding, dilation = _inputs(CASES["dilated_wide_pad"], torch.float16, seed=13)
    xd, wd, bd = x.to(device), wt.to(device), b.to(device)
    ref = _oracle(x, wt, b, stride, padding, dilation)
    out = torch.empty(ref.shape, dtype=x.dtype, device=device)
    a = _C.Conv2dArgs()
    a.input, a.weight, a.bias, a.output = xd.data_ptr(), wd.data_ptr(), bd.data_ptr(), out.data_ptr()
    a.batch, a.c_in, a.h_in, a.w_in = x.shape
    a.c_out, _, a.filter_h, a.filter_w = wt.shape
    (a.stride_h, a.stride_w), (a.pad_h, a.pad_w), (a.dil_h, a.dil_w) = stride, padding, dilation
    a.dtype = a.bias_dtype = _C.F16
    a.stream = torch.cuda.current_stream().cuda_stream
    assert _C.load().tnx_conv2d_forward(ctypes.byref(a)) == _C.OK        # block_* == 0: built-in choice
    torch.cuda.synchronize()
    assert oracle.within_tolerance(out, ref)[0]


def test_resnet_layer_at_size_against_the_vendor_routine_and_linearity(device):
    """Batch 32, 256 -> 256 channels, 56x56, 3x3: too large for the CPU oracle, so the checks are (i) sampled output
    planes against the oracle's fp32 library routine on the CPU, (ii) the vendor's GPU conv2d within the rounding
    of two bf16 results, (iii) conv(x, w1) + conv(x, w2) == conv(x, w1 + w2) when w1, w2 have disjoint support."""
    g = torch.Generator().manual_seed(21)
    x = torch.randn(32, 256, 56, 56, generator=g).bfloat16()
    wt = (torch.randn(256, 256, 3, 3, generator=g) / 48).bfloat16()
    b = torch.randn(256, generator=g).bfloat16()
    xd, wd, bd = x.to(device), wt.to(device), b.to(device)
    out = conv2d_forward(xd, wd, bd, (1, 1), (1, 1), (1, 1))
    regs = conv2d_forward(xd, wd, bd, (1, 1), (1, 1), (1, 1), config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64,
                                                                         LOADER="registers"))
    dma = conv2d_forward(xd, wd, bd, (1, 1), (1, 1), (1, 1), config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=256, BLOCK_SIZE_K=64,
                                                                        LOADER="dma"))
    assert torch.equal(regs, dma)
    for img in (0, 17, 31):
        ref = oracle.reference_conv2d(x[img:img + 1], wt, b, (1, 1), (1, 1), (1, 1))
        assert oracle.within_tolerance(out[img:img + 1], ref)[0]
    vendor = torch_conv2d_forward(xd, wd, bd, (1, 1), (1, 1), (1, 1))
    assert oracle.within_tolerance(out, vendor.float().cpu(), rel=2e-2)[0]
    mask = torch.zeros_like(wd)
    mask[:, :128] = 1
    y1 = conv2d_forward(xd, wd * mask, None, (1, 1), (1, 1), (1, 1)).float()
    y2 = conv2d_forward(xd, wd * (1 - mask), None, (1, 1), (1, 1), (1, 1)).float()
    y = conv2d_forward(xd, wd, None, (1, 1), (1, 1), (1, 1)).float()
    assert oracle.within_tolerance((y1 + y2).cpu(), y.cpu(), rel=2e-2)[0]


def test_zero_input_and_identity_filter(device):
    x = torch.zeros(2, 8, 9, 9, dtype=torch.bfloat16, device=device)
    wt = torch.randn(16, 8, 3, 3, device=device).bfloat16()
    b = torch.randn(16, device=device).bfloat16()
    out = conv2d_forward(x, wt, b, (1, 1), (1, 1), (1, 1), config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=32))
    assert torch.equal(out, b.view(1, 16, 1, 1).expand_as(out))
    # centre tap = identity matrix: the output is the input, bit for bit
    x = torch.randn(2, 16, 10, 12, device=device).bfloat16()
    wt = torch.zeros(16, 16, 3, 3, dtype=torch.bfloat16, device=device)
    wt[torch.arange(16), torch.arange(16), 1, 1] = 1
    out = conv2d_forward(x, wt, None, (1, 1), (1, 1), (1, 1), config=dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64))
    assert torch.equal(out, x)


# ---- float32 tensors: a three-term bf16 convolution over 3 c_in channels with an fp32 result ------------------
@pytest.mark.parametrize("name,config", [
    ("all_asymmetric", dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=32)),
    ("w_out_14", None),
    ("7x7_stem_ragged_k", dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64)),
    ("dilated_wide_pad", dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64)),
], ids=lambda v: str(v).replace(" ", "") if not isinstance(v, dict) else "tile%dx%d" % (v["BLOCK_SIZE_M"], v["BLOCK_SIZE_N"]))
def test_float32_conv2d(device, name, config, monkeypatch):
    """The reference convolves float32 tensors in TF32 (tritonix/ops/conv2d/forward.py:100-103, :231-236).  Here: fp32
    in, fp32 out, error against the float64 convolution far below a bf16 convolution's."""
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    x, wt, b, stride, padding, dilation = _inputs(CASES[name], torch.float32, seed=21)
    out = conv2d_forward(x.to(device), wt.to(device), None if b is None else b.to(device), stride, padding, dilation, config=config)
    assert out.dtype == torch.float32
    b64 = None if b is None else b.double()
    ref = torch.nn.functional.conv2d(x.double(), wt.double(), b64, stride, padding, dilation)
    err = ((out.cpu().double() - ref).abs().max() / ref.abs().max()).item()
    low = torch.nn.functional.conv2d(x.bfloat16().double(), wt.bfloat16().double(), b64, stride, padding, dilation)
    bf16 = ((low - ref).abs().max() / ref.abs().max()).item()
    assert err < 2e-4 and err * 30 < bf16, (err, bf16)
    assert oracle.within_tolerance(out, _oracle(x, wt, b, stride, padding, dilation))[0]


def test_float32_conv2d_1x1_on_the_gemm_route(device, monkeypatch):
    monkeypatch.setenv("TRITONIX_AUTOTUNE", "0")
    g = torch.Generator("cpu").manual_seed(23)
    x, wt, b = torch.randn(3, 96, 14, 14, generator=g), torch.randn(80, 96, 1, 1, generator=g) / 96 ** 0.5, torch.randn(80, generator=g)
    ref = torch.nn.functional.conv2d(x.double(), wt.double(), b.double())
    for loader in ("gemm", "registers", "auto"):
        cfg = dict(BLOCK_SIZE_M=0, BLOCK_SIZE_N=0, BLOCK_SIZE_K=0, LOADER=loader)
        out = conv2d_forward(x.to(device), wt.to(device), b.to(device), config=cfg)
        assert out.dtype == torch.float32
        assert ((out.cpu().double() - ref).abs().max() / ref.abs().max()).item() < 2e-4, loader


def test_float32_conv2d_on_the_direct_to_lds_kernel(device):
    """3 * 64 * 9 = 27 K slabs of 64: the split problem fits the DMA ring; same sums in the same order as the
    register-staged kernel, so the two float32 outputs agree bit for bit."""
    g = torch.Generator("cpu").manual_seed(31)
    x, wt, b = torch.randn(2, 64, 14, 14, generator=g), torch.randn(128, 64, 3, 3, generator=g) / 24, torch.randn(128, generator=g)
    xd, wd, bd = x.to(device), wt.to(device), b.to(device)
    tile = dict(BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, BLOCK_SIZE_K=64)
    dma = conv2d_forward(xd, wd, bd, (1, 1), (1, 1), (1, 1), config=dict(tile, LOADER="dma"))
    reg = conv2d_forward(xd, wd, bd, (1, 1), (1, 1), (1, 1), config=dict(tile, LOADER="registers"))
    assert dma.dtype == torch.float32 and torch.equal(dma, reg)
    ref = torch.nn.functional.conv2d(x.double(), wt.double(), b.double(), (1, 1), (1, 1))
    assert ((dma.cpu().double() - ref).abs().max() / ref.abs().max()).item() < 2e-4


def test_fp32_output_of_a_16_bit_convolution_rounds_to_the_16_bit_output(device):
    """`out_f32` hands out the fp32 sums (+ bias) before the one rounding: rounded here, they must be the bits the
    16-bit kernels write (register-staged kernel and GEMM route; through the C ABI)."""
    import ctypes

    from tritonix_amd import _C

    lib = _C.load()
    for name, loader in (("all_asymmetric", _C.CONV_LOADER_REGISTERS), ("3x3_same", _C.CONV_LOADER_REGISTERS), ("pointwise", _C.CONV_LOADER_GEMM)):
        if name == "pointwise":
            g = torch.Generator("cpu").manual_seed(29)
            x, wt, b = torch.randn(2, 64, 9, 9, generator=g).bfloat16(), (torch.randn(48, 64, 1, 1, generator=g) / 8).bfloat16(), torch.randn(48, generator=g).bfloat16()
            stride, padding, dilation = (1, 1), (0, 0), (1, 1)
        else:
            x, wt, b, stride, padding, dilation = _inputs(CASES[name], torch.bfloat16, seed=27)
        n, c, h, w = x.shape
        k, _, r, s = wt.shape
        ho, wo = conv.output_size(h, w, r, s, stride, padding, dilation)
        xd, wd, bd = x.to(device), wt.to(device), None if b is None else b.to(device)
        outs = {}
        for f32 in (0, 1):
            out = torch.empty(n, k, ho, wo, dtype=torch.float32 if f32 else torch.bfloat16, device=device)
            a = _C.Conv2dArgs()
            a.input, a.weight, a.output = xd.data_ptr(), wd.data_ptr(), out.data_ptr()
            a.bias = None if bd is None else bd.data_ptr()
            a.batch, a.c_in, a.h_in, a.w_in, a.c_out, a.filter_h, a.filter_w = n, c, h, w, k, r, s
            (a.stride_h, a.stride_w), (a.pad_h, a.pad_w), (a.dil_h, a.dil_w) = stride, padding, dilation
            a.dtype, a.bias_dtype, a.loader, a.out_f32 = _C.BF16, _C.BF16, loader, f32
            a.stream = torch.cuda.current_stream().cuda_stream
            assert lib.tnx_conv2d_forward(ctypes.byref(a)) == _C.OK, (name, f32)
            torch.cuda.synchronize()
            outs[f32] = out
        assert torch.equal(outs[1].bfloat16().view(torch.int16), outs[0].view(torch.int16)), name
