import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


def _have_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def default_library_options():
    """Every test starts from, and leaves behind, the library's default options
    (ccglib_amd.set_option), so that a test which selects a code path cannot leak
    its choice into the next one."""
    try:
        import ccglib_amd as cc
        defaults = {o: cc.get_option(o) for o in cc.Option}
    except (RuntimeError, OSError):
        yield          # library not built: tests that need it fail on their own
        return
    yield
    for o, v in defaults.items():
        cc.set_option(o, v)
