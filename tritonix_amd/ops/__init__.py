"""Operators built on the HIP tile kernels: GEMM / split-K GEMM (``matmul``), the gated GEMM (``swiglu``) and
conv2d forward (``conv2d``)."""
import importlib

# ``ops.matmul`` names both a module and, once imported, the dispatcher it defines: bind the names explicitly
_matmul_module = importlib.import_module("tritonix_amd.ops.matmul")
_swiglu_module = importlib.import_module("tritonix_amd.ops.swiglu")
_conv2d_module = importlib.import_module("tritonix_amd.ops.conv2d")

__all__ = []
for _module, _names in ((_matmul_module, ("matmul", "triton_matmul", "hip_matmul", "matmul_splitk", "matmul_kernel",
                                           "gemm_splitk_kernel")),
                        (_swiglu_module, ("glu_kernel", "swiglu_kernel", "glu", "swiglu", "swiglu_ffn", "fused_glu")),
                        (_conv2d_module, ("conv2d_forward", "conv2d_forward_kernel", "torch_conv2d_forward"))):
    for _name in _names:
        globals()[_name] = getattr(_module, _name)
        __all__.append(_name)
del _module, _names, _name
