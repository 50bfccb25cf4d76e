import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def built():
    """The in-tree native libraries; compiled only if nothing is there yet."""
    from fastmax_amd import _cabi, _ext

    if not (os.path.exists(_cabi.LIB_PATH) and os.path.exists(_ext.EXT_PATH)):
        from fastmax_amd import build

        build.build_all()
    return _cabi.load()


@pytest.fixture(autouse=True)
def kernel_path(request, monkeypatch):
    """Where the library has two kernel families for a shape (head dimensions 32 and 64: moment states, or
    dense score tiles for short sequences) FASTMAX_PATH picks one.  The test modules written against the
    moment kernels keep exercising them at every length; a module sets KERNEL_PATH = "dense" or "auto" to
    test the other family or the library's own choice."""
    path = getattr(request.module, "KERNEL_PATH", "moments")
    if path == "auto":
        monkeypatch.delenv("FASTMAX_PATH", raising=False)
    else:
        monkeypatch.setenv("FASTMAX_PATH", path)
