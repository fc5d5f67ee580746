"""The C-ABI library loads without a GPU and exports every symbol include/tah_duo.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tah_duo.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tah_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from tah_amd import _capi, _lib
    names = declared_symbols()
    assert "tah_duo_fwd_varlen" in names and "tah_duo_bwd_varlen" in names and "tah_duo_decode" in names
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/tah_duo.h but not exported by libtah_duo.so"
    assert sorted(_capi.PROTOTYPES) == names
    bound = _lib.lib()
    assert bound.tah_duo_abi_version() == _capi.ABI_VERSION
    assert bound.tah_duo_error_string(-2).decode().startswith("unsupported shape")


def test_struct_sizes_match_c_layout():
    """ctypes mirrors must have the sizes the C compiler gives the structs (LP64)."""
    from tah_amd import _capi
    assert ctypes.sizeof(_capi.DuoStream) == 9 * 8 + 8 * 8 + 2 * 4
    assert ctypes.sizeof(_capi.DuoFwdArgs) == 2 * ctypes.sizeof(_capi.DuoStream) + 4 * 4 + 4 + 4
    assert ctypes.sizeof(_capi.DuoBwdStream) == 5 * 8 + 8 * 8
    assert ctypes.sizeof(_capi.KvSegment) == 5 * 8 + 4 * 8 + 2 * 4


def test_product_ops_refuse_cpu_tensors():
    import pytest
    import torch

    from tah_amd import TahDuoError, ops
    with pytest.raises(TahDuoError):
        ops.hard_index_build(torch.zeros(2, 3, dtype=torch.bool))
