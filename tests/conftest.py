import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
# The reference's import line is `from ff_attention import FastForwardAttn`; the compiled
# module of that name lives in the package directory.
_EXT_DIR = os.path.join(ROOT, "fastforwardattention_amd")
if _EXT_DIR not in sys.path:
    sys.path.append(_EXT_DIR)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    from fastforwardattention_amd import _build
    _build.ensure_built()      # loads what is built; compiles only what is missing


def _have_gpu() -> bool:
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
