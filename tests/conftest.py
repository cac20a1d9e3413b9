import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are skipped (not failed) when no device is visible and the
    # user did not ask for them explicitly with -m gpu.
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def knobs():
    """knobs(nseg=2, prefix=1): set launch-heuristic overrides of the library for one test; every
    knob is back at -1 (the heuristic) afterwards."""
    from rfa_amd import _lib
    touched = []

    def set_(**kw):
        for name, value in kw.items():
            touched.append(name)
            _lib.tuning_set(name, value)
    yield set_
    for name in touched:
        _lib.tuning_set(name, -1)


@pytest.fixture(params=["ext", "ctypes"])
def binding(request):
    """Runs a test once through each binding of the kernel library: the PyTorch C++ extension and
    the ctypes wrappers (use with pytest.mark.usefixtures("binding"))."""
    from rfa_amd import rfa_hip
    if request.param == "ext" and not rfa_hip.ext_available():
        pytest.skip("the torch binding has not been built")
    before = rfa_hip.binding()
    rfa_hip.use_binding(request.param)
    yield request.param
    rfa_hip.use_binding(before)
