import json
import os
import sys
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# dispatcher records written by the tests stay out of the user's cache
os.environ.setdefault("TRITONIX_CACHE_DIR", tempfile.mkdtemp(prefix="tritonix_test_cache_"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load the library that is built; only when there is none do they build it (hipcc, a few minutes)."""
    from tritonix_amd import _C

    if not os.path.exists(_C.LIB_PATH):
        from tritonix_amd import build as hip_build

        hip_build.build(verbose=False)


@pytest.fixture(scope="session")
def traces():
    with open(os.path.join(ROOT, "tests", "golden", "hand_traces.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no HIP device visible")
    return torch.device("cuda", 0)
