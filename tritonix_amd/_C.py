"""ctypes binding of libtritonix_hip.so (the C ABI declared in include/tritonix_hip.h).

The library is built ahead of time by ``python -m tritonix_amd.build`` and is
loaded from the package directory.  There is no fallback: if it is missing,
every entry point raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

from tritonix_amd.testing import LDS_LIMIT_BYTES, OutOfResources

# TRITONIX_HIP_LIB names another build of the same library (development builds of a few tiles)
LIB_PATH = os.environ.get("TRITONIX_HIP_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)),
                                                              "libtritonix_hip.so")

# enum tnx_dtype
F16, BF16, I8, I32, F32 = 0, 1, 2, 3, 4
# enum tnx_epilogue
EPI_NONE, EPI_GLU_SILU, EPI_GLU_SIGMOID, EPI_GLU_IDENTITY = 0, 1, 2, 3
# enum tnx_schedule (flags)
SCHED_DEFAULT, SCHED_PERSISTENT, SCHED_SUPERBLOCK, SCHED_ATOMIC_REDUCE = 0, 1, 2, 4
# enum tnx_status
OK, E_INVALID, E_UNSUPPORTED, E_LDS, E_WORKSPACE, E_HIP, E_STATIC_LIMIT = 0, 1, 2, 3, 4, 5, 6
STATIC_WORKSPACE_BYTES = 65536 + (32 << 20)
# enum tnx_conv_loader
CONV_LOADER_AUTO, CONV_LOADER_REGISTERS, CONV_LOADER_DMA, CONV_LOADER_GEMM = 0, 1, 2, 3

EXPORTS = ("tnx_gemm", "tnx_gemm_static_workspace", "tnx_gemm_workspace_bytes", "tnx_gemm_lds_bytes", "tnx_gemm_supported",
           "tnx_gemm_default_config", "tnx_tile_coords", "tnx_split_f32", "tnx_kernel_count", "tnx_kernel_name", "tnx_strerror",
           "tnx_last_hip_error", "tnx_version", "tnx_conv2d_forward", "tnx_conv2d_supported", "tnx_conv2d_output_size",
           "tnx_conv2d_default_config", "tnx_conv2d_kernel_count", "tnx_conv2d_kernel_name")


class GemmArgs(ctypes.Structure):
    """struct tnx_gemm_args"""
    _fields_ = [
        ("a", ctypes.c_void_p), ("b", ctypes.c_void_p), ("c", ctypes.c_void_p),
        ("m", ctypes.c_int64), ("n", ctypes.c_int64), ("k", ctypes.c_int64),
        ("stride_am", ctypes.c_int64), ("stride_ak", ctypes.c_int64),
        ("stride_bk", ctypes.c_int64), ("stride_bn", ctypes.c_int64),
        ("stride_cm", ctypes.c_int64), ("stride_cn", ctypes.c_int64),
        ("in_dtype", ctypes.c_int32), ("out_dtype", ctypes.c_int32),
        ("block_m", ctypes.c_int32), ("block_n", ctypes.c_int32), ("block_k", ctypes.c_int32),
        ("group_m", ctypes.c_int32), ("split_k", ctypes.c_int32),
        ("num_stages", ctypes.c_int32), ("num_warps", ctypes.c_int32),
        ("epilogue", ctypes.c_int32), ("tail_tiles", ctypes.c_int32), ("schedule", ctypes.c_int32),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
    ]


class Conv2dArgs(ctypes.Structure):
    """struct tnx_conv2d_args"""
    _fields_ = [
        ("input", ctypes.c_void_p), ("weight", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("output", ctypes.c_void_p),
        ("batch", ctypes.c_int32), ("c_in", ctypes.c_int32), ("h_in", ctypes.c_int32), ("w_in", ctypes.c_int32),
        ("c_out", ctypes.c_int32), ("filter_h", ctypes.c_int32), ("filter_w", ctypes.c_int32),
        ("stride_h", ctypes.c_int32), ("stride_w", ctypes.c_int32), ("pad_h", ctypes.c_int32), ("pad_w", ctypes.c_int32),
        ("dil_h", ctypes.c_int32), ("dil_w", ctypes.c_int32),
        ("dtype", ctypes.c_int32), ("bias_dtype", ctypes.c_int32),
        ("block_pixels", ctypes.c_int32), ("block_cout", ctypes.c_int32), ("block_k", ctypes.c_int32),
        ("group_pixels", ctypes.c_int32), ("loader", ctypes.c_int32),
        ("stream", ctypes.c_void_p), ("out_f32", ctypes.c_int32),
    ]


_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m tritonix_amd.build` "
                           "(there is no non-HIP implementation to fall back to)")
    lib = ctypes.CDLL(LIB_PATH)
    p = ctypes.POINTER(GemmArgs)
    lib.tnx_gemm.argtypes = [p]
    lib.tnx_gemm.restype = ctypes.c_int
    lib.tnx_gemm_static_workspace.argtypes = [p]
    lib.tnx_gemm_static_workspace.restype = ctypes.c_int
    lib.tnx_gemm_workspace_bytes.argtypes = [p]
    lib.tnx_gemm_workspace_bytes.restype = ctypes.c_size_t
    lib.tnx_gemm_lds_bytes.argtypes = [p]
    lib.tnx_gemm_lds_bytes.restype = ctypes.c_int64
    lib.tnx_gemm_supported.argtypes = [p]
    lib.tnx_gemm_supported.restype = ctypes.c_int
    lib.tnx_gemm_default_config.argtypes = [p]
    lib.tnx_gemm_default_config.restype = ctypes.c_int
    lib.tnx_tile_coords.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_int)] * 2
    lib.tnx_tile_coords.restype = ctypes.c_int
    lib.tnx_split_f32.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                  ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p]
    lib.tnx_split_f32.restype = ctypes.c_int
    lib.tnx_kernel_count.argtypes = []
    lib.tnx_kernel_count.restype = ctypes.c_int
    lib.tnx_kernel_name.argtypes = [ctypes.c_int]
    lib.tnx_kernel_name.restype = ctypes.c_char_p
    lib.tnx_strerror.argtypes = [ctypes.c_int]
    lib.tnx_strerror.restype = ctypes.c_char_p
    lib.tnx_last_hip_error.argtypes = []
    lib.tnx_last_hip_error.restype = ctypes.c_int
    lib.tnx_version.argtypes = []
    lib.tnx_version.restype = ctypes.c_int
    cp = ctypes.POINTER(Conv2dArgs)
    for name in ("tnx_conv2d_forward", "tnx_conv2d_supported", "tnx_conv2d_default_config"):
        getattr(lib, name).argtypes = [cp]
        getattr(lib, name).restype = ctypes.c_int
    lib.tnx_conv2d_output_size.argtypes = [cp, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]
    lib.tnx_conv2d_output_size.restype = None
    lib.tnx_conv2d_kernel_count.argtypes = []
    lib.tnx_conv2d_kernel_count.restype = ctypes.c_int
    lib.tnx_conv2d_kernel_name.argtypes = [ctypes.c_int]
    lib.tnx_conv2d_kernel_name.restype = ctypes.c_char_p
    _lib = lib
    return lib


def strerror(status: int) -> str:
    return load().tnx_strerror(status).decode()


def raise_for_status(status: int, args: GemmArgs) -> None:
    """Map a tnx_status to the exception the tuner and the dispatcher expect."""
    if status == OK:
        return
    lib = load()
    if status == E_LDS:
        raise OutOfResources(int(lib.tnx_gemm_lds_bytes(ctypes.byref(args))), LDS_LIMIT_BYTES, "shared memory")
    if status == E_UNSUPPORTED:
        raise ValueError(
            f"{strerror(status)}: dtype={args.in_dtype} block=({args.block_m},{args.block_n},{args.block_k}) "
            f"warps={args.num_warps} stages={args.num_stages} split_k={args.split_k} epilogue={args.epilogue}")
    if status == E_HIP:
        raise RuntimeError(f"{strerror(status)} (hipError_t {lib.tnx_last_hip_error()})")
    if status in (E_WORKSPACE, E_STATIC_LIMIT):
        raise RuntimeError(strerror(status))
    raise ValueError(strerror(status))


def tile_coords(schedule: int, idx: int, tiles_m: int, tiles_n: int, group_m: int = 8):
    """(tile_m, tile_n) the workgroup with launch-order id ``idx`` computes under ``schedule`` (host arithmetic)."""
    tm, tn = ctypes.c_int(), ctypes.c_int()
    status = load().tnx_tile_coords(schedule, idx, tiles_m, tiles_n, group_m, ctypes.byref(tm), ctypes.byref(tn))
    if status != OK:
        raise ValueError(strerror(status))
    return tm.value, tn.value


def conv2d_kernel_names():
    lib = load()
    return [lib.tnx_conv2d_kernel_name(i).decode() for i in range(lib.tnx_conv2d_kernel_count())]


def kernel_names():
    lib = load()
    return [lib.tnx_kernel_name(i).decode() for i in range(lib.tnx_kernel_count())]
