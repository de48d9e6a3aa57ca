import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def km():
    """The ctypes plumbing over the C ABI (package directory has a hyphen, hence import_module)."""
    mod = importlib.import_module("cuda-kmeans_amd")
    if not os.path.exists(mod.HOST_LIB_PATH) or not os.path.exists(mod.HIP_LIB_PATH):
        mod.build(force=False)
    return mod


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    from oracle import binding
    binding.oracle_lib()
    return binding


@pytest.fixture(scope="session")
def gpu(km):
    """Device guard for the GPU tests: fails loudly (no skip, no fallback) when the card is missing."""
    assert km.device_count() > 0, "no HIP device visible: GPU tests must run on the MI355X box"
    km.check(km.hip_lib().kmx_set_device(0))
    return km.device_props()
