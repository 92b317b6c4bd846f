import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def hip_lib():
    """The built C-ABI library; compiled once here only when no built copy exists."""
    from twilight_amd import _lib, build
    if not os.path.exists(build.LIB_PATH):
        build.build_library()
    return _lib.lib()


@pytest.fixture(scope="session")
def dev(hip_lib):
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
