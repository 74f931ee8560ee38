"""The reference's import paths resolve to the HIP engine's modules (tritonix/__init__.py of this repository)."""
import sys

import pytest
import torch


def test_reference_import_lines_work():
    import tritonix
    import tritonix_amd
    from tritonix.autotune import Choice, PowerOfTwo, Range, TunableKernel, tunable          # noqa: F401
    from tritonix.dispatcher import DynamicDispatcher, dynamic_dispatch                       # noqa: F401
    from tritonix.ops.matmul import matmul, matmul_kernel, matmul_splitk, triton_matmul       # noqa: F401
    from tritonix.ops.swiglu import glu_kernel                                                # noqa: F401
    from tritonix.utils.pruners import CoordinateUnimodalFunction, MonotonicCascadeTrie       # noqa: F401
    from tritonix.utils.spaces import SpaceConfig                                             # noqa: F401

    assert tritonix.matmul is tritonix_amd.matmul and matmul is tritonix_amd.matmul
    assert tritonix.matmul_splitk is tritonix_amd.matmul_splitk
    assert tritonix.tunable is tritonix_amd.tunable and tritonix.glu_kernel is tritonix_amd.glu_kernel
    # one module object under two names: state (config memos, dispatcher cache) is shared, not duplicated
    assert sys.modules["tritonix.ops.matmul"] is sys.modules["tritonix_amd.ops.matmul"]
    assert sys.modules["tritonix.utils.pruners"] is sys.modules["tritonix_amd.utils.pruners"]
    assert isinstance(matmul_kernel, TunableKernel)


def test_conv2d_forward_import_lines_work():
    import tritonix
    import tritonix_amd
    from tritonix.ops.conv2d import conv2d_forward, conv2d_forward_kernel, torch_conv2d_forward   # noqa: F401
    from tritonix.ops.conv2d.forward import conv2d_forward as same

    assert tritonix.conv2d_forward is tritonix_amd.conv2d_forward is conv2d_forward is same
    assert tritonix.torch_conv2d_forward is torch_conv2d_forward


def test_operators_off_the_path_are_absent():
    with pytest.raises(ImportError):
        import tritonix.ops.statistics                                                        # noqa: F401
    with pytest.raises(ImportError):
        import tritonix.ops.conv2d.backward                                                   # noqa: F401
    import tritonix

    assert not hasattr(tritonix, "topk") and not hasattr(tritonix, "conv2d_grad_input_kernel")


def test_forced_oracle_backend_through_the_alias():
    import tritonix

    with tritonix.matmul.force_backend("pytorch"):
        out = tritonix.matmul(torch.ones(2, 3), torch.ones(3, 4))
    assert torch.equal(out, torch.full((2, 4), 3.0))


@pytest.mark.gpu
def test_matmul_through_the_reference_import_name(device):
    import oracle
    import tritonix

    a, b = oracle.make_inputs("C1")
    with tritonix.matmul.force_backend("triton"):
        out = tritonix.matmul(a.to(device), b.to(device))
    assert oracle.within_tolerance(out, oracle.reference_matmul(a, b))[0]
