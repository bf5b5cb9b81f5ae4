import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
# a test process: wrq_debug_override stays usable after the first launch (read by the library when it first looks)
os.environ.setdefault("WRQ_TEST_HOOKS", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import wrq_oracle

    wrq_oracle.lib()
    return wrq_oracle


@pytest.fixture(scope="session")
def wrq():
    import importlib

    return importlib.import_module("web-rwkv_amd")


@pytest.fixture(scope="session")
def gpu(wrq):
    """The binding with the library loaded on a real GPU; fails (never skips) without one."""
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    status = wrq.lib().wrq_init()
    assert status == 0, wrq.lib().wrq_last_error().decode()
    return wrq


@pytest.fixture
def overrides(wrq):
    """Pins kernel / tile choices through wrq_debug_override for one test; released afterwards."""
    used = set()

    def pin(**kv):
        for key, value in kv.items():
            wrq.debug_override(key, value)
            used.add(key)

    yield pin
    for key in used:
        wrq.debug_override(key, -1)
