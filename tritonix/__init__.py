"""``tritonix`` import name over the gfx950 engine.

Callers of the reference write ``import tritonix``, ``from tritonix.ops.matmul import matmul,
triton_matmul, matmul_kernel`` and ``from tritonix.autotune import tunable`` (tests/test_matmul.py:1-8,
examples/tune_matmul.py:1-10 of the reference).  This package maps those module paths onto the modules of
``tritonix_amd`` so such code runs unchanged on the HIP kernels: every ``tritonix.x.y`` below *is* the module
``tritonix_amd.x.y`` (one module object, two names), nothing is re-implemented here.

Only the dense tiled-GEMM path and conv2d forward exist: ``tritonix.ops.conv2d.backward``,
``tritonix.ops.statistics`` and the other operators of the reference are not provided and importing them raises
``ImportError``.
"""
import importlib
import sys

import tritonix_amd

_ALIASED = ("autotune", "dispatcher", "testing", "kernel", "ops", "ops.matmul", "ops.swiglu", "ops.conv2d",
            "ops.conv2d.forward", "utils", "utils.spaces", "utils.pruners")

for _name in _ALIASED:
    sys.modules[f"{__name__}.{_name}"] = importlib.import_module(f"tritonix_amd.{_name}")
for _name in ("autotune", "dispatcher", "testing", "kernel", "ops", "utils"):
    globals()[_name] = sys.modules[f"{__name__}.{_name}"]
del _name

# the names the reference's package exports for this path (tritonix/__init__.py:3-17)
from tritonix_amd import *  # noqa: E402,F401,F403
from tritonix_amd import __all__ as _amd_all, __version__  # noqa: E402,F401

__all__ = list(_amd_all)
