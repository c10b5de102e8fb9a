import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _library_knobs_follow_environment():
    """Tests change TRITEIA_HIP_* variables through `monkeypatch`; the library snapshots them, so it is told to
    read them again once the test's changes have been undone (autouse fixtures are set up first and torn down
    last, i.e. after monkeypatch has restored the environment)."""
    yield
    try:
        from triteia_amd.python.capi import _ffi
        if os.path.exists(_ffi.LIB_PATH):
            _ffi.reload_env()
    except Exception:
        pass
