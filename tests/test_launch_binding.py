"""Host side of a launch: how a Triton-style call (tritonix/ops/matmul.py:222-236, :249-263; tritonix/ops/swiglu.py:24-43)
is bound to one ``tnx_gemm_args``.  No GPU: nothing is launched, and launching without one must fail loudly."""
import ctypes

import pytest
import torch

import tritonix_amd
from tritonix_amd import _C
from tritonix_amd.kernel import HipKernel


def call(kernel, a, b, c, **kw):
    m, k = a.shape
    n = b.shape[1]
    return kernel._bind((a, b, c, m, n, k, a.stride(0), a.stride(1), b.stride(0), b.stride(1), c.stride(0), c.stride(1)), kw)


TILE = dict(block_m=128, block_n=128, block_k=64, group_m=8, num_stages=2, num_warps=4)


def tensors(dtype=torch.bfloat16, m=256, n=384, k=512):
    return torch.zeros(m, k, dtype=dtype), torch.zeros(k, n, dtype=dtype), torch.zeros(m, n, dtype=dtype)


def test_arguments_land_in_the_struct():
    a, b, c = tensors()
    g = tritonix_amd.matmul_kernel.make_args(call(tritonix_amd.matmul_kernel, a, b, c, **TILE))
    assert (g.m, g.n, g.k) == (256, 384, 512)
    assert (g.stride_am, g.stride_ak, g.stride_bk, g.stride_bn, g.stride_cm, g.stride_cn) == (512, 1, 384, 1, 384, 1)
    assert (g.in_dtype, g.out_dtype) == (_C.BF16, _C.BF16)
    assert (g.block_m, g.block_n, g.block_k, g.group_m, g.num_stages, g.num_warps) == (128, 128, 64, 8, 2, 4)
    assert (g.split_k, g.tail_tiles, g.epilogue, g.schedule) == (1, 0, _C.EPI_NONE, 0)
    assert (g.a, g.b, g.c) == (a.data_ptr(), b.data_ptr(), c.data_ptr())
    assert _C.load().tnx_gemm_supported(ctypes.byref(g)) == _C.OK


def test_transposed_views_keep_their_strides():
    a, b, c = tensors()
    bt = torch.zeros(384, 512, dtype=torch.bfloat16).t()                 # [k, n] view of an [n, k] tensor
    g = tritonix_amd.matmul_kernel.make_args(call(tritonix_amd.matmul_kernel, a, bt, c, **TILE))
    assert (g.stride_bk, g.stride_bn) == (1, 512)
    assert _C.load().tnx_gemm_supported(ctypes.byref(g)) == _C.OK          # the element-wise loader takes it


def test_k_cut_keywords_are_optional_everywhere():
    a, b, c = tensors()
    for kernel in (tritonix_amd.matmul_kernel, tritonix_amd.glu_kernel):
        g = kernel.make_args(call(kernel, a, b, c, split_k=4, tail_tiles=3, **TILE))
        assert (g.split_k, g.tail_tiles) == (4, 3)
    g = tritonix_amd.gemm_splitk_kernel.make_args(call(tritonix_amd.gemm_splitk_kernel, a, b, c, split_k=2, **TILE))
    assert (g.split_k, g.tail_tiles) == (2, 0)
    with pytest.raises(TypeError):                                       # split_k is part of this kernel's signature
        call(tritonix_amd.gemm_splitk_kernel, a, b, c, **TILE)


def test_glu_activation_mapping():
    a, b, c = tensors()
    z = torch.zeros(256, 192, dtype=torch.bfloat16)
    k = tritonix_amd.glu_kernel
    assert k.make_args(call(k, a, b, z, **TILE)).epilogue == _C.EPI_GLU_SILU                     # default, as in the reference
    assert k.make_args(call(k, a, b, z, activation="sigmoid", **TILE)).epilogue == _C.EPI_GLU_SIGMOID
    # any other value leaves the gate un-activated (tritonix/ops/swiglu.py:100-102)
    assert k.make_args(call(k, a, b, z, activation="relu", **TILE)).epilogue == _C.EPI_GLU_IDENTITY
    assert k.make_args(call(k, a, b, z, use_tf32=False, **TILE)).epilogue == _C.EPI_GLU_SILU


def test_bad_calls_raise_type_errors():
    a, b, c = tensors()
    k = tritonix_amd.matmul_kernel
    with pytest.raises(TypeError, match="missing"):
        call(k, a, b, c, block_m=128)
    with pytest.raises(TypeError, match="unexpected"):
        call(k, a, b, c, num_ctas=2, **TILE)
    with pytest.raises(TypeError, match="multiple values"):
        k._bind((a, b, c, 1, 2, 3, 4, 5, 6, 7, 8, 9, 128), dict(TILE))
    with pytest.raises(ValueError, match="share a dtype"):
        k.make_args(call(k, a, b.to(torch.float16), c, **TILE))
    with pytest.raises(ValueError, match="no HIP kernel"):
        k.make_args(call(k, a.double(), b.double(), c.double(), **TILE))
    # fp32 has a dtype code (split-K slices are fp32) but no kernel takes it as an input
    g = k.make_args(call(k, a.float(), b.float(), c.float(), **TILE))
    assert _C.load().tnx_gemm_supported(ctypes.byref(g)) == _C.E_INVALID


def test_int8_accumulates_into_int32():
    a, b, _ = tensors(torch.int8)
    c = torch.zeros(256, 384, dtype=torch.int32)
    g = tritonix_amd.matmul_kernel.make_args(call(tritonix_amd.matmul_kernel, a, b, c, **dict(TILE, block_k=128)))
    assert (g.in_dtype, g.out_dtype) == (_C.I8, _C.I32)
    assert _C.load().tnx_gemm_supported(ctypes.byref(g)) == _C.OK
    g.out_dtype = _C.I8
    assert _C.load().tnx_gemm_supported(ctypes.byref(g)) == _C.E_UNSUPPORTED


def test_there_is_no_cpu_path():
    """Host tensors are refused: the package has no implementation besides the HIP kernels."""
    a, b, c = tensors()
    with pytest.raises(ValueError, match="HIP device"):
        tritonix_amd.matmul_kernel[(2, 3)](a, b, c, 256, 384, 512, 512, 1, 384, 1, 384, 1, **TILE)
    with pytest.raises(ValueError, match="HIP device"):
        tritonix_amd.gemm_splitk_kernel[(2, 3, 2)](a, b, c, 256, 384, 512, 512, 1, 384, 1, 384, 1, split_k=2, **TILE)


def test_new_kernel_objects_follow_the_same_protocol():
    k = HipKernel("probe", ["block_m", "block_n", "block_k", "group_m", "num_stages", "num_warps"])
    assert k.arg_names[:12] == ["a", "b", "c", "m", "n", "k", "stride_am", "stride_ak", "stride_bk", "stride_bn",
                                "stride_cm", "stride_cn"]
    assert k.arg_names[-5:] == ["split_k", "tail_tiles", "persistent", "superblock", "atomic_reduce"]
    seen = []
    k.add_pre_run_hook(lambda *a, **kw: seen.append(kw.get("block_m")))
    a, b, c = tensors()
    with pytest.raises(ValueError):
        k[(1,)](a, b, c, 256, 384, 512, 512, 1, 384, 1, 384, 1, **TILE)
    assert seen == []                                                   # hooks run only for launches that can happen


def test_swiglu_kernel_keeps_the_reference_signature():
    """``swiglu_kernel[grid](x, w12, w3, z, m, n, k, f, 8 strides, block_m=, block_n=, block_k=, group_m=, block_l=,
    use_tf32=, activation=)`` (tritonix/ops/swiglu.py:127-152), exported as the reference exports it
    (tritonix/__init__.py:15)."""
    from tritonix.ops.swiglu import glu_kernel, swiglu_kernel                                # noqa: F401
    import tritonix

    assert tritonix.swiglu_kernel is tritonix_amd.swiglu_kernel is swiglu_kernel
    assert isinstance(swiglu_kernel, tritonix_amd.TunableKernel)
    assert swiglu_kernel.arg_names[:16] == ["x", "w12", "w3", "z", "m", "n", "k", "f", "stride_xm", "stride_xk", "stride_wk",
                                            "stride_wn", "stride_w3n", "stride_w3l", "stride_zm", "stride_zl"]
    assert swiglu_kernel.arg_names[16:23] == ["block_m", "block_n", "block_k", "group_m", "block_l", "use_tf32", "activation"]
    assert swiglu_kernel.keys == ["m", "n", "k"] and swiglu_kernel.specialize_keys == ["m", "n", "k"]
    assert list(swiglu_kernel.space) == ["block_m", "block_n", "block_k", "block_l", "group_m", "num_stages", "num_warps"]
    assert {"block_m", "block_n", "block_k", "block_l", "num_stages"} <= swiglu_kernel.memory_params
    x, w12, w3 = torch.zeros(128, 256, dtype=torch.bfloat16), torch.zeros(256, 512, dtype=torch.bfloat16), torch.zeros(256, 192, dtype=torch.bfloat16)
    z = torch.zeros(128, 192, dtype=torch.bfloat16)
    pos = (x, w12, w3, z, 128, 512, 256, 192, 256, 1, 512, 1, 192, 1, 192, 1)
    tile = dict(block_m=128, block_n=128, block_k=64, group_m=8, block_l=64, num_stages=2, num_warps=4)
    bound = swiglu_kernel._bind(pos, dict(tile, activation="sigmoid"))
    assert bound["f"] == 192 and bound["stride_w3n"] == 192 and bound["block_l"] == 64 and bound["activation"] == "sigmoid"
    with pytest.raises(TypeError, match="missing"):
        swiglu_kernel._bind(pos, dict(block_m=128))
    with pytest.raises(TypeError, match="unexpected"):
        swiglu_kernel._bind(pos, dict(tile, num_ctas=1))
    with pytest.raises(ValueError, match="HIP device"):                  # no CPU path here either
        swiglu_kernel[(1, 4)](*pos, **tile)


def test_workspace_handed_out_under_graph_capture_is_never_released(monkeypatch):
    """A captured launch bakes its split-K workspace pointer into the graph: neither the LRU eviction nor a later,
    larger request may free that buffer (bookkeeping only; no GPU)."""
    from tritonix_amd import kernel

    dev = torch.device("cpu", 0)
    monkeypatch.setattr(kernel, "_workspaces", type(kernel._workspaces)())
    monkeypatch.setattr(kernel, "_captured_workspaces", [])
    monkeypatch.setattr(kernel, "_capturing", lambda: True)
    captured = kernel._workspace(dev, 1, 1 << 20)
    assert kernel._workspace(dev, 1, 1 << 20) is captured and len(kernel._captured_workspaces) == 1
    monkeypatch.setattr(kernel, "_capturing", lambda: False)
    grown = kernel._workspace(dev, 1, 4 << 20)                           # a later launch needs more: a new buffer
    assert grown is not captured and grown.numel() >= 4 << 20
    for stream in range(2, 2 + 2 * kernel._MAX_WORKSPACES):                # ... and many other streams push it out of the LRU
        kernel._workspace(dev, stream, 16)
    assert len(kernel._workspaces) == kernel._MAX_WORKSPACES
    assert any(kept is captured for kept in kernel._captured_workspaces)  # still alive for the graph's replays


def test_float32_calls_are_rewritten_as_a_three_term_bf16_product():
    """float32 operands (the reference multiplies them in TF32, tritonix/ops/matmul.py:98) become a bf16 problem with
    k' = 3k and an fp32 result on a tile of at most 128x128; no kernel takes float32 itself."""
    from tritonix_amd.ops.matmul import default_config

    a, b = torch.zeros(300, 200), torch.zeros(200, 520)
    cfg = default_config(a, b)
    assert cfg["block_m"] * cfg["block_n"] <= 128 * 128
    g = _C.GemmArgs()
    g.m, g.n, g.k = 300, 520, 600
    g.stride_am, g.stride_ak, g.stride_bk, g.stride_bn, g.stride_cm, g.stride_cn = 600, 1, 520, 1, 520, 1
    g.in_dtype, g.out_dtype = _C.BF16, _C.F32
    g.block_m, g.block_n, g.block_k, g.group_m, g.num_stages, g.num_warps = 128, 128, 64, 8, 3, 8
    g.split_k = 1
    lib = _C.load()
    assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.OK
    g.epilogue = _C.EPI_GLU_SILU
    assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.OK                # the gated epilogue writes fp32 too
    g.epilogue = _C.EPI_NONE
    g.block_m, g.block_n, g.num_stages, g.num_warps = 256, 256, 2, 4       # no fp32 epilogue in the large tiles
    assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.E_UNSUPPORTED
    g.block_m, g.block_n, g.block_k, g.num_stages, g.num_warps = 128, 128, 128, 2, 4
    g.in_dtype = _C.I8
    assert lib.tnx_gemm_supported(ctypes.byref(g)) == _C.E_UNSUPPORTED     # int8 accumulates into int32 only
    # argument checks of the splitter run on the host
    assert lib.tnx_split_f32(None, 4, 4, 4, 1, None, 0, None) == _C.E_INVALID
    assert lib.tnx_split_f32(None, 0, 4, 4, 1, None, 0, None) == _C.OK     # nothing to do
    assert lib.tnx_split_f32(None, 4, 4, 4, 1, None, 2, None) == _C.E_INVALID
    assert lib.tnx_split_f32(None, -1, 4, 4, 1, None, 0, None) == _C.E_INVALID
