import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped (not failed) where no GPU is visible."""
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def ob():
    from oracle import binding
    binding.lib()
    return binding


@pytest.fixture(scope="session")
def ref(ob):
    r = ob.ref()
    if r is None:
        pytest.skip("oracle/_ref/libmcnref.so has not been built (needs the MatConvNet sources)")
    return ob


@pytest.fixture(scope="session")
def capi():
    from matconvnet_amd import capi as c
    c.lib()  # raises if the HIP library is missing: there is no fallback
    return c


@pytest.fixture(scope="session")
def vl():
    from matconvnet_amd import vlapi
    vlapi.lib()  # raises if the C++ operator library is missing: there is no fallback
    return vlapi
