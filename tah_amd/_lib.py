"""Loads the PyTorch-ROCm extension (``tah_amd._C``, built in-tree from csrc/torch_ext.cpp) and has it open the
MI355X library (``libtah_duo.so``, the C ABI of include/tah_duo.h).

There is no fallback: if either is missing, every op of this package raises.  Build both with
``make -C tah_amd/csrc`` (or ``python -c 'import __graft_entry__ as g; g.build()'`` from the repo root).
"""
from __future__ import annotations

import os

from . import _capi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtah_duo.so")
_ext = None


def ext():
    """The extension module, without loading a library into it."""
    global _ext
    if _ext is None:
        try:
            import torch  # noqa: F401  (the extension links against libtorch)

            from . import _C
        except ImportError as e:
            raise _capi.TahDuoError(
                f"the PyTorch extension tah_amd._C is not built ({e}); run `make -C tah_amd/csrc`; "
                "tah_amd has no CPU or PyTorch fallback") from None
        _ext = _C
    return _ext


def lib():
    """The extension with libtah_duo.so loaded (loads it on first use)."""
    e = ext()
    if not e.loaded():
        if not os.path.exists(LIB_PATH):
            raise _capi.TahDuoError(
                f"{LIB_PATH} not found: the HIP library is not built (run `make -C tah_amd/csrc`); "
                "tah_amd has no CPU or PyTorch fallback")
        try:
            e.load_library(LIB_PATH, False)
        except RuntimeError as err:
            raise _capi.TahDuoError(str(err)) from None
    return e
