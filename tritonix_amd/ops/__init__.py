from tritonix_amd.ops.matmul import (matmul, triton_matmul, hip_matmul, matmul_splitk, matmul_kernel,
                                     gemm_splitk_kernel)
from tritonix_amd.ops.swiglu import glu_kernel, glu, swiglu, swiglu_ffn, fused_glu

__all__ = ["matmul", "triton_matmul", "hip_matmul", "matmul_splitk", "matmul_kernel", "gemm_splitk_kernel",
           "glu_kernel", "glu", "swiglu", "swiglu_ffn", "fused_glu"]
