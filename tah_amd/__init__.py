"""MI355X-native duo-causal attention for Think-at-Hard (TaH).

Hand-written HIP kernels for gfx950 behind a C ABI (include/tah_duo.h), bound to
torch tensors by a PyTorch-ROCm C++ extension (tah_amd._C), with a Python host
layer that mirrors the reference's attention / KV-cache / hard-token pack
interfaces.  There is no CPU or PyTorch fallback.
"""
from . import _capi, _lib, ops  # noqa: F401
from ._capi import TahDuoError  # noqa: F401

__all__ = ["ops", "TahDuoError"]
