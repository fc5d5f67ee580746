"""Loads the MI355X duo-causal attention library (libtah_duo.so, built in-tree).

There is no fallback: if the library is missing or cannot be loaded, every op of
this package raises.  Build it with ``make -C tah_amd/csrc`` (or
``python -c 'import __graft_entry__ as g; g.build()'`` from the repo root).
"""
from __future__ import annotations

import ctypes
import os

from . import _capi

_HERE = os.path.dirname(os.path.abspath(__file__))
# TAH_DUO_LIB: developer override naming another build of the same library (kernel tuning).
LIB_PATH = os.environ.get("TAH_DUO_LIB") or os.path.join(_HERE, "libtah_duo.so")
_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise _capi.TahDuoError(
                f"{LIB_PATH} not found: the HIP library is not built (run `make -C tah_amd/csrc`); "
                "tah_amd has no CPU or PyTorch fallback")
        _lib = _capi.bind(ctypes.CDLL(LIB_PATH))
    return _lib
