"""Loads the CPU execution build of the HIP kernels (tah_amd/csrc/emu) for tests.

The kernels' sources are compiled unchanged with the host clang++ against a shim
``hip/hip_runtime.h`` that runs every GPU thread as an OS thread.  This checks a
kernel's indexing, masking, LDS layout and barrier placement without a GPU.  It
is test infrastructure: the package never loads this library.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "tah_amd", "csrc")
HOSTCXX = "/opt/rocm/lib/llvm/bin/clang++"


def have_host_clang() -> bool:
    return os.path.exists(HOSTCXX)


def build(san: str = "") -> str:
    name = {"": "libtah_duo_emu.so", "address": "libtah_duo_emu_asan.so", "thread": "libtah_duo_emu_tsan.so"}[san]
    out = os.path.join(CSRC, "emu", name)
    srcs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith((".hip", ".h"))]
    srcs += [os.path.join(CSRC, "emu", "hip", "hip_runtime.h"), os.path.join(ROOT, "include", "tah_duo.h")]
    if os.path.exists(out) and all(os.path.getmtime(out) >= os.path.getmtime(s) for s in srcs):
        return out
    cmd = ["make", "-s", "-C", CSRC, "emu", f"EMU_OUT=emu/{name}"]
    if san:
        cmd.append(f"EMU_SAN=-fsanitize={san}")
    subprocess.check_call(cmd)
    return out


@contextlib.contextmanager
def emulated():
    """Have the package's extension open the CPU execution build (and accept host tensors) for the duration of
    the block; afterwards it opens the MI355X library again.  Yields the same library bound with ctypes, for
    tests that call the C ABI directly."""
    from tah_amd import _capi, _lib

    path = build()
    ext = _lib.ext()
    ext.load_library(path, True)
    try:
        yield _capi.bind(ctypes.CDLL(path))
    finally:
        ext.load_library(_lib.LIB_PATH, False)
