import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_present():
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker (tests only)."""
    import oracle as module

    return module


@pytest.fixture(scope="session")
def library():
    """libsphericart_amd.so through ctypes; built beforehand, never here on a GPU box."""
    from sphericart_amd import _c_lib

    if not os.path.exists(_c_lib.LIBRARY_PATH):
        from sphericart_amd.build import build

        build()
    return _c_lib.get_library()


@pytest.fixture
def switches(library):
    """Override planning decisions of the library for one test (sphx_set_switch); all overrides
    are dropped afterwards."""

    def set_switch(name, value):
        assert library.sphx_set_switch(name.encode(), int(value)) == 0, library.sphx_last_error()

    library.sphx_reset_switches()
    yield set_switch
    library.sphx_reset_switches()


def same_numbers(a, b):
    """Element-wise identity as numbers: equal values (so -0.0 == 0.0) or NaN in both."""
    a = np.asarray(a)
    b = np.asarray(b)
    return (a == b) | (np.isnan(a) & np.isnan(b))
