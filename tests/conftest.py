import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# The drop-in Python package lives under the (non-importable, hyphenated)
# project folder; tests import it the way a user of the original would.
for p in (ROOT, os.path.join(ROOT, "deformable-kernels_amd"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def switch_off():
    """`switch_off("DK_NO_MFMA", ...)` switches the named kernel families of the library off (its test
    hook dk_test_switches) until the test ends, so that the next more general kernels serve the call."""
    from deformable_kernels.ops.deform_kernel import _lib
    before = _lib.lib().dk_test_switches(0)
    _lib.lib().dk_test_switches(before)
    active = [before]

    def off(*names):
        for n in names:
            active[0] |= 1 << _lib.TEST_SWITCHES.index(n)
        _lib.lib().dk_test_switches(active[0])

    yield off
    _lib.lib().dk_test_switches(before)
