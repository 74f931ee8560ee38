"""tritonix_amd: the dense tiled-GEMM path of tritonix on hand-written gfx950 (MI355X) HIP kernels.

Same Python surface as the reference package (tritonix/__init__.py): ``matmul``,
``matmul_splitk``, ``tunable`` / ``TunableKernel`` / ``PowerOfTwo`` / ``Range`` /
``Choice``, ``glu_kernel``, ``swiglu_kernel``, ``conv2d_forward`` / ``torch_conv2d_forward``, plus the host
wrappers ``glu`` / ``swiglu``.
"""
from tritonix_amd.autotune import tunable, TunableKernel, PowerOfTwo, Range, Choice, OutOfResources
from tritonix_amd.dispatcher import DynamicDispatcher, dynamic_dispatch
from tritonix_amd.ops.matmul import (matmul, triton_matmul, hip_matmul, matmul_splitk, matmul_kernel,
                                     gemm_splitk_kernel)
from tritonix_amd.ops.swiglu import glu_kernel, swiglu_kernel, glu, swiglu, swiglu_ffn, fused_glu
from tritonix_amd.ops.conv2d import conv2d_forward, conv2d_forward_kernel, torch_conv2d_forward
from tritonix_amd.utils.spaces import SpaceConfig, ConfigSpace
from tritonix_amd.utils.pruners import (MonotonicCascadeTrie, CoordinateUnimodalFunction,
                                        CoordinateMonotonicFunction)

__version__ = "0.1.0"

__all__ = ["matmul", "triton_matmul", "hip_matmul", "matmul_splitk", "matmul_kernel", "gemm_splitk_kernel",
           "glu_kernel", "swiglu_kernel", "glu", "swiglu", "swiglu_ffn", "fused_glu", "conv2d_forward", "conv2d_forward_kernel",
           "torch_conv2d_forward", "tunable", "TunableKernel", "PowerOfTwo", "Range", "Choice",
           "OutOfResources", "DynamicDispatcher", "dynamic_dispatch", "SpaceConfig", "ConfigSpace",
           "MonotonicCascadeTrie", "CoordinateUnimodalFunction", "CoordinateMonotonicFunction"]
