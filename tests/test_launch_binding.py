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
