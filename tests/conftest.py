import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def rt():
    """The process-wide HIP runtime of the library (GPU tests only)."""
    import arcinferzero_amd as az
    az.Runtime.init(0)
    print(f"[arcz] device: {az.Runtime.device_name()}, {az.Runtime.cus()} CUs", flush=True)
    yield az.Runtime
