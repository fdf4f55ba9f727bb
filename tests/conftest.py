import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, where no GPU is visible."""
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _automatic_conv_kernel_after_every_test():
    """The kernel choice of tab_set_conv_kernel is process-wide: whatever a test selected (and however it ended),
    the next test starts from the library's own choice."""
    yield
    try:
        from tab_amd import _capi
        lib = _capi.load()
    except Exception:  # library not built: the tests that need it fail on their own
        return
    lib.tab_set_conv_kernel(0, -1)
