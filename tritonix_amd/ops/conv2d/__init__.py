"""Conv2d forward as an implicit GEMM on the HIP tile engine (the reference's ``tritonix.ops.conv2d`` forward half)."""
from tritonix_amd.ops.conv2d.forward import conv2d_forward, conv2d_forward_kernel, torch_conv2d_forward

__all__ = ["conv2d_forward", "conv2d_forward_kernel", "torch_conv2d_forward"]
