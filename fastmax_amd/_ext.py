"""Loader of the in-tree PyTorch extension `fastmax_cuda` (built by fastmax_amd.build)."""
from __future__ import annotations

import importlib.util
import os
import sys
import sysconfig

_HERE = os.path.dirname(os.path.abspath(__file__))
EXT_PATH = os.path.join(_HERE, "fastmax_cuda" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))
_mod = None


def load():
    """The extension module; raises if it has not been built (there is no fallback)."""
    global _mod
    if _mod is None:
        import torch  # noqa: F401  (the extension links against libtorch)

        if not os.path.exists(EXT_PATH):
            raise RuntimeError(f"{EXT_PATH} is missing: build it with `python -m fastmax_amd.build`")
        spec = importlib.util.spec_from_file_location("fastmax_cuda", EXT_PATH)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _mod = mod
    return _mod


def install_as_fastmax_cuda():
    """Registers the extension as the top-level module `fastmax_cuda`, the name the reference's
    Python files import (example.py:4, model.py:18, test_fastmax.py:7)."""
    sys.modules["fastmax_cuda"] = load()
    return sys.modules["fastmax_cuda"]
