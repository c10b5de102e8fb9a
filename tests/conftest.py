import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "perf: wall-clock comparisons on a real MI355X; run only when asked for by name "
                                       "(-m perf): a noisy machine must not turn the parity suite red")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    asked_for_perf = "perf" in (config.getoption("-m") or "")
    not_asked = pytest.mark.skip(reason="timing test: runs only under -m perf")
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "perf" in item.keywords and not asked_for_perf:
            item.add_marker(not_asked)
        elif not have_gpu and ("gpu" in item.keywords or "perf" in item.keywords):
            item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def _library_is_built():
    """The tests load the library that is built in the tree and compile it only if there is none
    (hipcc cross-compiles without a GPU)."""
    from triteia_amd import build as _build
    _build.ensure_built(verbose=False)


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
