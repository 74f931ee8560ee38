"""Host side of the conv2d forward path: C-ABI argument checks, the built-in tile choice, the launch object's
argument binding (no GPU: nothing here launches)."""
import ctypes

import pytest
import torch

import oracle
from tritonix_amd import _C
from tritonix_amd.ops.conv2d import forward as conv


def _args(**kw):
    a = _C.Conv2dArgs()
    base = dict(batch=2, c_in=16, h_in=14, w_in=14, c_out=32, filter_h=3, filter_w=3, stride_h=1, stride_w=1, pad_h=1,
                pad_w=1, dil_h=1, dil_w=1, dtype=_C.BF16, bias_dtype=_C.BF16)
    base.update(kw)
    for k, v in base.items():
        setattr(a, k, v)
    return a


def test_output_size_matches_the_oracle_and_the_python_mirror():
    lib = _C.load()
    for (h, w, r, s, st, pd, dl) in [(224, 224, 7, 7, (2, 2), (3, 3), (1, 1)), (10, 13, 3, 2, (2, 1), (0, 2), (1, 2)),
                                     (7, 7, 3, 3, (1, 1), (0, 0), (2, 2)), (2, 2, 5, 5, (1, 1), (0, 0), (1, 1))]:
        a = _args(h_in=h, w_in=w, filter_h=r, filter_w=s, stride_h=st[0], stride_w=st[1], pad_h=pd[0], pad_w=pd[1],
                  dil_h=dl[0], dil_w=dl[1])
        ho, wo = ctypes.c_int32(), ctypes.c_int32()
        lib.tnx_conv2d_output_size(ctypes.byref(a), ctypes.byref(ho), ctypes.byref(wo))
        assert (ho.value, wo.value) == oracle.conv2d_output_size(h, w, r, s, st, pd, dl) == conv.output_size(h, w, r, s, st, pd, dl)


def test_supported_statuses():
    lib = _C.load()
    assert lib.tnx_conv2d_supported(ctypes.byref(_args())) == _C.OK                       # built-in tile
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_pixels=64, block_cout=64, block_k=32))) == _C.OK
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_pixels=96, block_cout=64, block_k=32))) == _C.E_UNSUPPORTED
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_pixels=512, block_cout=512, block_k=64))) == _C.E_LDS
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(dtype=_C.F32))) == _C.E_UNSUPPORTED
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(dtype=_C.I8))) == _C.E_INVALID
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(stride_h=0))) == _C.E_INVALID
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(pad_w=-1))) == _C.E_INVALID
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(h_in=2, w_in=2, filter_h=5, filter_w=5, pad_h=0, pad_w=0))) == _C.E_INVALID
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(h_in=20000))) == _C.E_UNSUPPORTED
    # more than 2^31 input elements
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(batch=4096, c_in=1024, h_in=64, w_in=64))) == _C.E_UNSUPPORTED
    assert lib.tnx_conv2d_supported(None) == _C.E_INVALID


def test_forward_rejects_null_pointers_before_launching():
    assert _C.load().tnx_conv2d_forward(ctypes.byref(_args())) == _C.E_INVALID


def test_default_config_names_a_built_tile():
    lib = _C.load()
    built = set(_C.conv2d_kernel_names())
    assert len(built) >= 16
    gemm_tiles = {tuple(name.split()[:4]) for name in _C.kernel_names()}
    loaders = {_C.CONV_LOADER_REGISTERS: "registers", _C.CONV_LOADER_DMA: "dma", _C.CONV_LOADER_GEMM: "gemm"}
    one_by_one = dict(filter_h=1, filter_w=1, pad_h=0, pad_w=0)
    seen = set()
    for kw in (dict(), dict(c_out=512, c_in=512, batch=32), dict(c_out=8, c_in=3, **one_by_one),
               dict(batch=1, h_in=4, w_in=4), dict(c_in=64, c_out=256, h_in=56, w_in=56, batch=32),
               dict(c_in=64, c_out=128, h_in=28, w_in=28, batch=8), dict(c_in=64, c_out=128, stride_w=2),
               dict(c_in=64, c_out=256, h_in=56, w_in=56, batch=32, **one_by_one),
               dict(c_in=1024, c_out=256, h_in=14, w_in=14, batch=32, **one_by_one),
               dict(c_in=100, c_out=256, h_in=14, w_in=14, batch=32, **one_by_one)):
        a = _args(**kw)
        assert lib.tnx_conv2d_default_config(ctypes.byref(a)) == _C.OK
        if a.loader == _C.CONV_LOADER_GEMM:
            assert ("bf16", str(a.block_cout), str(a.block_pixels), str(a.block_k)) in gemm_tiles
        else:
            assert f"bf16 {a.block_cout} {a.block_pixels} {a.block_k} {loaders[a.loader]}" in built
        assert a.group_pixels == 8
        assert lib.tnx_conv2d_supported(ctypes.byref(a)) == _C.OK
        seen.add((a.block_cout, a.block_pixels, loaders[a.loader]))
    # c_in * 9 a multiple of 64 and unit stride along w: the direct-to-LDS kernel; 256 channels wide when that leaves
    # two tiles per CU
    assert (256, 128, "dma") in seen and (128, 128, "dma") in seen and (128, 64, "registers") in seen
    # 1x1 layers with unit stride and no padding: the GEMM route
    assert (128, 128, "gemm") in seen and (64, 64, "gemm") in seen
    for kw in (dict(c_in=1024, c_out=256, h_in=14, w_in=14, batch=32), dict(c_in=3, c_out=8), dict(c_in=64, c_out=64, h_in=7, w_in=7)):
        a = _args(**kw, **one_by_one)
        assert lib.tnx_conv2d_default_config(ctypes.byref(a)) == _C.OK and a.loader == _C.CONV_LOADER_GEMM
    a = _args(c_in=64, c_out=64, stride_h=2, **one_by_one)
    assert lib.tnx_conv2d_default_config(ctypes.byref(a)) == _C.OK and a.loader != _C.CONV_LOADER_GEMM


def test_loader_requests():
    lib = _C.load()
    ok = dict(c_in=64, c_out=128, block_pixels=128, block_cout=128, block_k=64)
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=_C.CONV_LOADER_DMA, **ok))) == _C.OK
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=_C.CONV_LOADER_REGISTERS, **ok))) == _C.OK
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=4, **ok))) == _C.E_INVALID
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=-1, **ok))) == _C.E_INVALID
    # stride along w, or c_in * R * S not a multiple of 64: only the register-staged kernel
    for bad in (dict(stride_w=2), dict(c_in=16)):
        kw = dict(ok, **bad)
        assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=_C.CONV_LOADER_DMA, **kw))) == _C.E_UNSUPPORTED
        assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=_C.CONV_LOADER_AUTO, **kw))) == _C.OK
    # a tile only one of the two kernels has
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=_C.CONV_LOADER_DMA, c_in=64, block_pixels=64, block_cout=64,
                                                       block_k=64))) == _C.E_UNSUPPORTED


def test_gemm_route_requests():
    """The GEMM route serves 1x1 filters with unit stride and no padding, on any built GEMM tile or its own choice."""
    lib = _C.load()
    flat = dict(filter_h=1, filter_w=1, pad_h=0, pad_w=0, loader=_C.CONV_LOADER_GEMM)
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(**flat))) == _C.OK
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(c_in=7, h_in=5, w_in=3, c_out=5, **flat))) == _C.OK
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_cout=128, block_pixels=128, block_k=64, **flat))) == _C.OK
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_cout=64, block_pixels=128, block_k=32, **flat))) == _C.OK
    # the 256-wide GEMM tiles carry no problem index and no bias
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_cout=256, block_pixels=256, block_k=64, **flat))) == _C.E_UNSUPPORTED
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(dil_h=3, dil_w=2, **flat))) == _C.OK     # one tap: dilation has no effect
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_cout=96, block_pixels=128, block_k=64, **flat))) == _C.E_UNSUPPORTED
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(block_cout=128, block_pixels=0, block_k=64, **flat))) == _C.E_UNSUPPORTED
    for bad in (dict(filter_h=3, pad_h=1), dict(stride_h=2), dict(stride_w=2), dict(pad_w=1)):
        assert lib.tnx_conv2d_supported(ctypes.byref(_args(**dict(flat, **bad)))) == _C.E_UNSUPPORTED
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=_C.CONV_LOADER_GEMM))) == _C.E_UNSUPPORTED   # the 3x3 default
    # a caller's tile with "auto" names a conv2d kernel, never the GEMM route: a tile only the GEMM kernels have is refused
    only_gemm = dict(block_cout=32, block_pixels=64, block_k=64, c_in=64, filter_h=1, filter_w=1, pad_h=0, pad_w=0)
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(**only_gemm))) == _C.E_UNSUPPORTED
    assert lib.tnx_conv2d_supported(ctypes.byref(_args(loader=_C.CONV_LOADER_GEMM, **only_gemm))) == _C.OK


def test_every_reference_candidate_is_built():
    built = set(_C.conv2d_kernel_names())
    for bm, bn, bk, _ in conv._CANDIDATE_CONFIGS:
        for dt in ("bf16", "f16"):
            assert f"{dt} {bn} {bm} {bk} registers" in built
    for dt in ("bf16", "f16"):
        for bc, bp in ((128, 128), (256, 128), (128, 256)):
            assert f"{dt} {bc} {bp} 64 dma" in built


def test_candidate_filter_follows_the_reference():
    # tritonix/ops/conv2d/forward.py:243-254: tiles wider than the problem are dropped once the problem has 64 rows/columns
    c = conv.candidate_configs(gemm_m=100, gemm_n=64, gemm_k=48)
    assert all(bm <= 100 and bn <= 64 and bk <= 48 for bm, bn, bk, _ in c) and c
    assert conv.candidate_configs(gemm_m=10, gemm_n=10, gemm_k=8) == [(64, 64, 32, 8)]
    # below 64 the size filter does not apply
    assert (128, 128, 32, 8) in conv.candidate_configs(gemm_m=10, gemm_n=10, gemm_k=32)


def _call(x, w, out, bias=None, **over):
    n, c, h, wd = x.shape
    k, _, r, s = w.shape
    ho, wo = conv.output_size(h, wd, r, s, (1, 1), (1, 1), (1, 1))
    vals = dict(output_ptr=out, input_ptr=x, weight_ptr=w, bias_ptr=bias, BATCH_SIZE=n, C_IN=c, H_IN=h, W_IN=wd, C_OUT=k,
                H_OUT=ho, W_OUT=wo, FILTER_H=r, FILTER_W=s, stride_h=1, stride_w=1, pad_h=1, pad_w=1, dil_h=1, dil_w=1,
                GEMM_M=n * ho * wo, GEMM_N=k, GEMM_K=c * r * s)
    vals.update(over)
    pos = [vals[n_] for n_ in conv.conv2d_forward_kernel.arg_names]
    return conv.conv2d_forward_kernel.bind(*pos, BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=32, GROUP_SIZE_M=8,
                                           USE_TF32=True)


def test_launch_object_binds_the_reference_argument_order(monkeypatch):
    class _S:
        cuda_stream = 0
    monkeypatch.setattr(torch.cuda, "current_stream", lambda device=None: _S())
    x = torch.zeros(2, 4, 6, 6, dtype=torch.bfloat16)
    w = torch.zeros(8, 4, 3, 3, dtype=torch.bfloat16)
    out = torch.zeros(2, 8, 6, 6, dtype=torch.bfloat16)
    b = torch.zeros(8, dtype=torch.float32)
    a = _call(x, w, out, b)
    assert (a.batch, a.c_in, a.h_in, a.w_in, a.c_out, a.filter_h, a.filter_w) == (2, 4, 6, 6, 8, 3, 3)
    assert (a.block_pixels, a.block_cout, a.block_k, a.group_pixels) == (64, 64, 32, 8)
    assert a.input == x.data_ptr() and a.weight == w.data_ptr() and a.output == out.data_ptr() and a.bias == b.data_ptr()
    assert a.dtype == _C.BF16 and a.bias_dtype == _C.F32
    assert _call(x, w, out).bias is None
    with pytest.raises(ValueError):
        _call(x, w, out, H_OUT=5)
    with pytest.raises(ValueError):
        _call(x, w, out, GEMM_K=7)
    with pytest.raises(ValueError):
        _call(x, w, out.half())
    with pytest.raises(ValueError):
        _call(x.permute(0, 1, 3, 2).contiguous().permute(0, 1, 3, 2), w, out)      # not contiguous NCHW
    with pytest.raises(TypeError):
        conv.conv2d_forward_kernel.bind(out, x, w)


def test_conv2d_forward_argument_errors():
    x = torch.zeros(1, 4, 6, 6, dtype=torch.bfloat16)
    w = torch.zeros(8, 4, 3, 3, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        conv.conv2d_forward(x.permute(0, 1, 3, 2), w)
    with pytest.raises(AssertionError):
        conv.conv2d_forward(x, torch.zeros(8, 5, 3, 3, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="HIP device"):                # host tensors: there is no CPU path, float32 included
        conv.conv2d_forward(x.float(), w.float(), config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64))
    with pytest.raises(ValueError, match="HIP device"):
        conv.conv2d_forward(x, w, config=dict(BLOCK_SIZE_M=64, BLOCK_SIZE_N=64, BLOCK_SIZE_K=64))


def test_torch_conv2d_forward_is_the_library_routine():
    g = torch.Generator().manual_seed(0)
    x, w, b = torch.randn(1, 2, 5, 5, generator=g), torch.randn(3, 2, 3, 3, generator=g), torch.randn(3, generator=g)
    got = conv.torch_conv2d_forward(x, w, b, (2, 1), (1, 0), (1, 1))
    assert torch.equal(got, torch.nn.functional.conv2d(x, w, b, (2, 1), (1, 0), (1, 1)))
