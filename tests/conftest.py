import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # PyTorch carries its own copy of the HIP runtime. A process that loads libyvex_rocm.so (and
    # with it the system's copy) before torch ends up with two runtimes, and the second one finds
    # no device: torch goes first in every test process, also for tests that never touch it.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass


@pytest.fixture(scope="session")
def oracle():
    import oracle as module
    module.build()
    return module


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    from yvex_amd import load_library
    load_library()   # raises if the HIP library is not built: no fallback exists
    return torch.device("cuda:0")
