"""MI355X-native decode attention with FastForwardAttention's extension API.

    from fastforwardattention_amd import FastForwardAttn          # or: from ff_attention import ...
    ffa = FastForwardAttn(K, V, prompt_len + output_len, use_default_kernel_launch)
    out = ffa.attention(q, k, v, softmax_scale, t, p)

`FastForwardAttn` is the pybind11 class of the compiled extension `ff_attention`
(csrc/torch_ffa_api.cpp), which calls the C ABI of include/ffa_c_api.h implemented by
libffa_hip.so (hand-written gfx950 kernels).  There is no Python or CPU fallback: if the
compiled parts are missing, importing the class raises ImportError.  Build them with
`python -m fastforwardattention_amd._build`.

`fastforwardattention_amd.capi` binds the same C ABI with ctypes for callers that hold raw
device pointers.
"""
from __future__ import annotations

import importlib
import os
import sys

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))

__all__ = ["FastForwardAttn", "ff_attention", "capi"]


def _load_extension():
    """Load the compiled module once, under the reference's top-level name `ff_attention`
    (so that `from ff_attention import FastForwardAttn` and this package share one module
    object and one pybind11 type registration)."""
    if "ff_attention" in sys.modules:
        return sys.modules["ff_attention"]
    try:
        import torch  # noqa: F401  (libtorch must be loaded before the extension)
        sys.path.insert(0, _PKG_DIR)
        try:
            return importlib.import_module("ff_attention")
        finally:
            sys.path.remove(_PKG_DIR)
    except ImportError as exc:
        raise ImportError(
            "fastforwardattention_amd: the compiled extension ff_attention (and libffa_hip.so) "
            "is not built or cannot be loaded; run `python -m fastforwardattention_amd._build`. "
            f"Original error: {exc}") from exc


def __getattr__(name):
    # Lazy so that `import fastforwardattention_amd._build` works before anything is built.
    if name == "ff_attention":
        return _load_extension()
    if name == "FastForwardAttn":
        return __getattr__("ff_attention").FastForwardAttn
    if name == "capi":
        return importlib.import_module("fastforwardattention_amd.capi")
    raise AttributeError(name)
