import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "mini-caffe_amd"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu_mode():
    """Puts the calling thread in HIP mode; GPU tests depend on this fixture."""
    import minicaffe as mc
    assert mc.check_gpu_available(), "GPU test selected but no HIP device is visible"
    mc.set_runtime_mode(1, 0)
    return mc
