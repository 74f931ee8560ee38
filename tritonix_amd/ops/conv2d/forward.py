"""conv2d forward over the HIP implicit-GEMM kernel, with the reference's calling surface.

``conv2d_forward(input, weight, bias, stride, padding, dilation, use_tf32, config)`` and the launch
``conv2d_forward_kernel[grid](out, input, weight, bias, N, C_IN, H_IN, W_IN, C_OUT, H_OUT, W_OUT, R, S, str_h,
str_w, pad_h, pad_w, dil_h, dil_w, GEMM_M, GEMM_N, GEMM_K, BLOCK_SIZE_M=, BLOCK_SIZE_N=, BLOCK_SIZE_K=,
GROUP_SIZE_M=, OUT_DTYPE=, USE_TF32=)`` keep the argument order and meaning of
tritonix/ops/conv2d/forward.py:19-48 and :202-311; both end in one ``tnx_conv2d_forward`` through the C ABI on
torch's current stream.  Float16 and bfloat16 are built; float32 tensors (the reference convolves them in TF32,
which gfx950 has no matrix instruction for) run as a three-term bf16 convolution over 3 c_in channels with an fp32
result (``_split_f32``), on the register-staged kernels and the 1x1 GEMM route.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional, Tuple

import torch

from tritonix_amd import _C
from tritonix_amd.kernel import cdiv

__all__ = ["conv2d_forward", "conv2d_forward_kernel", "torch_conv2d_forward", "output_size", "candidate_configs"]

_DTYPES = {torch.float16: _C.F16, torch.bfloat16: _C.BF16, torch.float32: _C.F32}

# (BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K, GROUP_SIZE_M): the reference's candidates
# (tritonix/ops/conv2d/forward.py:172-180) and three larger tiles this engine also builds
_CANDIDATE_CONFIGS = [
    (128, 128, 32, 8),
    (128, 64, 32, 8),
    (64, 128, 32, 8),
    (64, 64, 32, 8),
    (128, 128, 64, 8),
    (64, 128, 64, 8),
    (128, 64, 64, 8),
    (64, 64, 64, 8),
    (64, 256, 64, 8),
    (128, 256, 64, 8),
    (256, 128, 64, 8),
]
_CONV_FWD_CONFIG_CACHE: Dict[tuple, dict] = {}
# optional launch keyword LOADER (no counterpart in the reference): which of the two kernels moves the slabs
_LOADERS = {"auto": _C.CONV_LOADER_AUTO, "registers": _C.CONV_LOADER_REGISTERS, "dma": _C.CONV_LOADER_DMA,
            "gemm": _C.CONV_LOADER_GEMM}


def output_size(h_in: int, w_in: int, filter_h: int, filter_w: int, stride, padding, dilation) -> Tuple[int, int]:
    """(H_OUT, W_OUT) as tritonix/ops/conv2d/forward.py:226-227 computes them."""
    h_out = (h_in + 2 * padding[0] - dilation[0] * (filter_h - 1) - 1) // stride[0] + 1
    w_out = (w_in + 2 * padding[1] - dilation[1] * (filter_w - 1) - 1) // stride[1] + 1
    return h_out, w_out


def _split_f32(x, w, batch, c_in, h_in, w_in, c_out, filter_h, filter_w):
    """float32 input and weight as the bf16 tensors of a three-term product (the reference convolves float32 in
    TF32, tritonix/ops/conv2d/forward.py:100-103; gfx950 has no TF32 matrix instruction): both are cut into a bf16 head
    and tail along the input channels, ``x -> [hi | hi | lo]`` (3 c_in channels) and ``w -> [hi | lo | hi]``, so that the
    ordinary bf16 convolution over 3 c_in channels with an fp32 result is ``hi hi + hi lo + lo hi``.  Returns
    ``(x3, w3, 3 * c_in)``."""
    lib = _C.load()
    stream = torch.cuda.current_stream(x.device).cuda_stream
    x3 = torch.empty((batch, 3 * c_in, h_in, w_in), dtype=torch.bfloat16, device=x.device)
    w3 = torch.empty((c_out, 3 * c_in, filter_h, filter_w), dtype=torch.bfloat16, device=x.device)
    for src, rows, cols, dst, side in ((x, batch, c_in * h_in * w_in, x3, 0), (w, c_out, c_in * filter_h * filter_w, w3, 2)):
        status = lib.tnx_split_f32(src.data_ptr(), rows, cols, cols, 1, dst.data_ptr(), side, stream)
        if status != _C.OK:
            raise RuntimeError(f"tnx_split_f32: {_C.strerror(status)}")
    return x3, w3, 3 * c_in


def _raise_for_status(status: int, a: _C.Conv2dArgs) -> None:
    if status == _C.OK:
        return
    lib = _C.load()
    if status == _C.E_UNSUPPORTED:
        if a.dtype == _C.F32:
            raise NotImplementedError("conv2d_forward is built for float16 and bfloat16; float32 (TF32) input has no "
                                      "matrix instruction on gfx950")
        raise ValueError(f"{_C.strerror(status)}: conv2d dtype={a.dtype} BLOCK_SIZE_M={a.block_pixels} "
                         f"BLOCK_SIZE_N={a.block_cout} BLOCK_SIZE_K={a.block_k}")
    if status == _C.E_LDS:
        raise _C.OutOfResources(2 * 2 * a.block_k * (a.block_pixels + a.block_cout), _C.LDS_LIMIT_BYTES, "shared memory")
    if status == _C.E_HIP:
        raise RuntimeError(f"{_C.strerror(status)} (hipError_t {lib.tnx_last_hip_error()})")
    raise ValueError(f"{_C.strerror(status)}: conv2d")


def _args(out, input, weight, bias, batch, c_in, h_in, w_in, c_out, filter_h, filter_w, stride, padding, dilation,
          block_m: int, block_n: int, block_k: int, group_m: int, loader: int = 0) -> _C.Conv2dArgs:
    a = _C.Conv2dArgs()
    if input.dtype == torch.float32:
        if not (input.is_cuda and weight.is_cuda and out.is_cuda):
            raise ValueError("conv2d_forward: input, weight and output must be tensors on a HIP device (there is no CPU path)")
        input, weight, c_in = _split_f32(input, weight, batch, c_in, h_in, w_in, c_out, filter_h, filter_w)
        a.out_f32 = 1
        a._keep = (input, weight)              # the scratch operands live as long as the bound arguments
    a.input, a.weight, a.output = input.data_ptr(), weight.data_ptr(), out.data_ptr()
    a.bias = bias.data_ptr() if bias is not None else None
    a.batch, a.c_in, a.h_in, a.w_in = batch, c_in, h_in, w_in
    a.c_out, a.filter_h, a.filter_w = c_out, filter_h, filter_w
    a.stride_h, a.stride_w = stride
    a.pad_h, a.pad_w = padding
    a.dil_h, a.dil_w = dilation
    if input.dtype not in _DTYPES:
        raise ValueError(f"conv2d_forward: dtype {input.dtype} has no HIP kernel (float16, bfloat16 and float32 are built)")
    a.dtype = _DTYPES[input.dtype]
    if bias is not None:
        if bias.dtype not in _DTYPES:
            raise ValueError(f"conv2d_forward: bias dtype {bias.dtype} is not a float type")
        a.bias_dtype = _DTYPES[bias.dtype]
    a.block_pixels, a.block_cout, a.block_k, a.group_pixels = block_m, block_n, block_k, group_m
    a.loader = loader
    a.stream = torch.cuda.current_stream(input.device).cuda_stream
    return a


class _Conv2dLaunch:
    def __init__(self, kernel, grid):
        self.kernel, self.grid = kernel, grid

    def __call__(self, *args, **kwargs):
        return self.kernel.run(*args, grid=self.grid, **kwargs)


class Conv2dForwardKernel:
    """``conv2d_forward_kernel[grid](...)`` with the reference's arguments (tritonix/ops/conv2d/forward.py:19-48).

    ``grid`` is accepted for compatibility; the engine derives its own 1-D grid.  H_OUT, W_OUT and the three GEMM
    sizes are checked against the values the other arguments imply.  ``OUT_DTYPE`` must be the input's type
    (it always is in the reference's host code, :231-236); ``USE_TF32`` is accepted and has no effect on 16-bit
    inputs."""

    arg_names = ("output_ptr", "input_ptr", "weight_ptr", "bias_ptr", "BATCH_SIZE", "C_IN", "H_IN", "W_IN", "C_OUT",
                 "H_OUT", "W_OUT", "FILTER_H", "FILTER_W", "stride_h", "stride_w", "pad_h", "pad_w", "dil_h", "dil_w",
                 "GEMM_M", "GEMM_N", "GEMM_K")

    def __getitem__(self, grid) -> _Conv2dLaunch:
        return _Conv2dLaunch(self, grid)

    def bind(self, *args, **kwargs) -> _C.Conv2dArgs:
        if len(args) > len(self.arg_names):
            raise TypeError(f"conv2d_forward_kernel takes {len(self.arg_names)} positional arguments, got {len(args)}")
        b = dict(zip(self.arg_names, args))
        for k, v in kwargs.items():
            if k in b:
                raise TypeError(f"conv2d_forward_kernel got multiple values for argument '{k}'")
            b[k] = v
        missing = [n for n in self.arg_names if n not in b and n != "bias_ptr"]
        missing += [n for n in ("BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K", "GROUP_SIZE_M") if n not in b]
        if missing:
            raise TypeError(f"conv2d_forward_kernel missing arguments: {', '.join(missing)}")
        out, x, w, bias = b["output_ptr"], b["input_ptr"], b["weight_ptr"], b.get("bias_ptr")
        stride, padding, dilation = (b["stride_h"], b["stride_w"]), (b["pad_h"], b["pad_w"]), (b["dil_h"], b["dil_w"])
        h_out, w_out = output_size(b["H_IN"], b["W_IN"], b["FILTER_H"], b["FILTER_W"], stride, padding, dilation)
        if (b["H_OUT"], b["W_OUT"]) != (h_out, w_out):
            raise ValueError(f"H_OUT, W_OUT = {b['H_OUT']}, {b['W_OUT']} do not follow from the other sizes ({h_out}, {w_out})")
        if (b["GEMM_M"], b["GEMM_N"], b["GEMM_K"]) != (b["BATCH_SIZE"] * h_out * w_out, b["C_OUT"],
                                                       b["C_IN"] * b["FILTER_H"] * b["FILTER_W"]):
            raise ValueError("GEMM_M, GEMM_N, GEMM_K do not follow from the other sizes")
        if not (x.is_contiguous() and w.is_contiguous() and out.is_contiguous()):
            raise ValueError("conv2d_forward_kernel addresses contiguous NCHW / KCRS tensors")
        if x.numel() != b["BATCH_SIZE"] * b["C_IN"] * b["H_IN"] * b["W_IN"] or \
                w.numel() != b["C_OUT"] * b["C_IN"] * b["FILTER_H"] * b["FILTER_W"] or \
                out.numel() != b["BATCH_SIZE"] * b["C_OUT"] * h_out * w_out or \
                (bias is not None and bias.numel() != b["C_OUT"]):
            raise ValueError("tensor sizes do not match the size arguments")
        if w.dtype != x.dtype or out.dtype != x.dtype:
            raise ValueError("input, weight and output must share one dtype")
        if bias is not None and not bias.is_contiguous():
            raise ValueError("bias must be contiguous")
        return _args(out, x, w, bias, b["BATCH_SIZE"], b["C_IN"], b["H_IN"], b["W_IN"], b["C_OUT"], b["FILTER_H"],
                     b["FILTER_W"], stride, padding, dilation, b["BLOCK_SIZE_M"], b["BLOCK_SIZE_N"], b["BLOCK_SIZE_K"],
                     b["GROUP_SIZE_M"], _LOADERS[b.get("LOADER", "auto")])

    def run(self, *args, grid=None, **kwargs):
        for t in args[:3]:
            if isinstance(t, torch.Tensor) and not t.is_cuda:
                raise ValueError("conv2d_forward_kernel: output, input and weight must be tensors on a HIP device (there is no CPU path)")
        a = self.bind(*args, **kwargs)
        _raise_for_status(_C.load().tnx_conv2d_forward(ctypes.byref(a)), a)

    def prepare(self, *args, **kwargs):
        """Bind once, launch many times: a callable that re-issues the same ``tnx_conv2d_forward`` (on the stream that
        was current when ``prepare`` ran)."""
        a = self.bind(*args, **kwargs)
        if a.out_f32:
            raise ValueError("conv2d_forward_kernel.prepare binds 16-bit launches; a float32 call splits its operands on every launch")
        fn = _C.load().tnx_conv2d_forward
        ref = ctypes.byref(a)

        def launch():
            status = fn(ref)
            if status != _C.OK:
                _raise_for_status(status, a)

        launch.args = a
        return launch

    def __repr__(self):
        return "<HipKernel conv2d_forward_kernel>"


conv2d_forward_kernel = Conv2dForwardKernel()


def candidate_configs(gemm_m: int, gemm_n: int, gemm_k: int):
    """The candidates the reference's mini-tuner times for a problem (tritonix/ops/conv2d/forward.py:243-254)."""
    out = []
    for bm, bn, bk, g in _CANDIDATE_CONFIGS:
        if bm > gemm_m and gemm_m >= 64:
            continue
        if bn > gemm_n and gemm_n >= 64:
            continue
        if bk > gemm_k:
            continue
        out.append((bm, bn, bk, g))
    if not out:
        out = [(64, 64, 32, 8)]
    return out


def _time_kernel(fn, iters=10, warmup=5, regions=3):
    """Mean launch time in ms: the fastest of `regions` event-timed runs of `iters` launches (one short region, as the
    reference times its candidates, picks a different tile from run to run on layers of a few tens of microseconds)."""
    for _ in range(warmup):
        fn()
    best = float("inf")
    for _ in range(regions):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        end.synchronize()
        best = min(best, start.elapsed_time(end) / iters)
    return best


def conv2d_forward(
    input: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    stride: Tuple[int, int] = (1, 1),
    padding: Tuple[int, int] = (0, 0),
    dilation: Tuple[int, int] = (1, 1),
    use_tf32: bool = True,
    config: Optional[dict] = None,
) -> torch.Tensor:
    """conv2d forward on the HIP kernel; same arguments and result as tritonix/ops/conv2d/forward.py:202-311.

    ``config=None`` times the candidate tiles once per problem key and remembers the fastest, as the reference
    does (with ``TRITONIX_AUTOTUNE=0`` in the environment it launches the library's built-in choice instead); ``config={"BLOCK_SIZE_M", "BLOCK_SIZE_N", "BLOCK_SIZE_K"[, "GROUP_SIZE_M"][, "LOADER"]}`` launches that tile
    (all three sizes 0: the library's own choice; ``LOADER`` is "auto", "registers", "dma" or "gemm").
    Returns a new [N, C_OUT, H_OUT, W_OUT] tensor of the input's dtype."""
    assert input.is_contiguous(), "Input must be contiguous NCHW"
    assert weight.is_contiguous(), "Weight must be contiguous KCRS"
    n, c_in, h_in, w_in = input.shape
    c_out, c_in_w, r, s = weight.shape
    assert c_in == c_in_w
    stride, padding, dilation = tuple(stride), tuple(padding), tuple(dilation)
    h_out, w_out = output_size(h_in, w_in, r, s, stride, padding, dilation)
    gemm_m, gemm_n, gemm_k = n * h_out * w_out, c_out, c_in * r * s
    out = input.new_empty((n, c_out, h_out, w_out))

    def launch(bm, bn, bk, g, loader="auto", dst=out):
        conv2d_forward_kernel[(cdiv(gemm_m, bm or 1), cdiv(gemm_n, bn or 1))](
            dst, input, weight, bias, n, c_in, h_in, w_in, c_out, h_out, w_out, r, s,
            stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], gemm_m, gemm_n, gemm_k,
            BLOCK_SIZE_M=bm, BLOCK_SIZE_N=bn, BLOCK_SIZE_K=bk, GROUP_SIZE_M=g, USE_TF32=use_tf32, LOADER=loader)

    if config is None and os.environ.get("TRITONIX_AUTOTUNE", "1") in ("0", "false", "False"):
        config = dict(BLOCK_SIZE_M=0, BLOCK_SIZE_N=0, BLOCK_SIZE_K=0)      # no timing runs: the library's own choice
    if config is None:
        key = (n, c_in, h_in, w_in, c_out, r, s, stride, padding, dilation, input.dtype)
        cfg = _CONV_FWD_CONFIG_CACHE.get(key)
        if cfg is None:
            best_time, best = float("inf"), None
            for bm, bn, bk, g in candidate_configs(gemm_m, gemm_n, gemm_k):
                try:
                    t = _time_kernel(lambda: launch(bm, bn, bk, g))
                except (ValueError, _C.OutOfResources):
                    continue
                if t < best_time:
                    best_time, best = t, dict(BLOCK_SIZE_M=bm, BLOCK_SIZE_N=bn, BLOCK_SIZE_K=bk, GROUP_SIZE_M=g)
            if (r, s) == (1, 1) and stride == (1, 1) and padding == (0, 0):
                # a 1x1 layer is a plain GEMM per image: the library's GEMM route with its own tile is one more candidate
                try:
                    t = _time_kernel(lambda: launch(0, 0, 0, 8, "gemm"))
                    if t < best_time:
                        best_time, best = t, dict(BLOCK_SIZE_M=0, BLOCK_SIZE_N=0, BLOCK_SIZE_K=0, GROUP_SIZE_M=8, LOADER="gemm")
                except (ValueError, _C.OutOfResources):
                    pass
            if best is None:
                raise RuntimeError("conv2d_forward: no candidate tile could be launched")
            _CONV_FWD_CONFIG_CACHE[key] = cfg = best
    else:
        cfg = config
    launch(cfg["BLOCK_SIZE_M"], cfg["BLOCK_SIZE_N"], cfg["BLOCK_SIZE_K"], cfg.get("GROUP_SIZE_M", 8), cfg.get("LOADER", "auto"))
    return out


def torch_conv2d_forward(
    input: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    stride: Tuple[int, int] = (1, 1),
    padding: Tuple[int, int] = (0, 0),
    dilation: Tuple[int, int] = (1, 1),
) -> torch.Tensor:
    """PyTorch's conv2d on the same arguments (tritonix/ops/conv2d/forward.py:314-323): the vendor baseline."""
    return torch.nn.functional.conv2d(input, weight, bias, stride, padding, dilation)
