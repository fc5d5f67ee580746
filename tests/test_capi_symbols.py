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
    bound = _capi.bind(lib)
    assert bound.tah_duo_abi_version() == _capi.ABI_VERSION
    assert bound.tah_duo_error_string(-2).decode().startswith("unsupported shape")


def test_torch_extension_loads_the_library_and_exposes_every_op():
    """The PyTorch extension (the binding the package uses) opens libtah_duo.so without a GPU, agrees on the ABI
    version and has one function per compute entry point of the header."""
    from tah_amd import _capi, _lib
    ext = _lib.lib()
    assert ext.loaded() and ext.abi_version() == _capi.ABI_VERSION
    for n in ("duo_fwd_varlen", "duo_bwd_varlen", "duo_fwd_masked", "duo_bwd_masked", "duo_decode", "decode_workspace_bytes",
              "kv_append", "qk_prep", "hard_index_build", "pad_rows_build", "rows_copy", "topk_mix", "sample_rows", "qk_prep_bwd", "silu_mul"):
        assert callable(getattr(ext, n))


def test_struct_sizes_match_c_layout(tmp_path):
    """ctypes mirrors must have the sizes the C compiler gives the structs of the header (gcc, LP64)."""
    import shutil
    import subprocess

    from tah_amd import _capi
    pairs = {"tah_duo_stream": _capi.DuoStream, "tah_duo_fwd_args": _capi.DuoFwdArgs, "tah_duo_bwd_stream": _capi.DuoBwdStream,
             "tah_duo_bwd_args": _capi.DuoBwdArgs, "tah_duo_schedule_args": _capi.DuoScheduleArgs, "tah_kv_segment": _capi.KvSegment,
             "tah_duo_decode_args": _capi.DuoDecodeArgs, "tah_qk_prep_args": _capi.QkPrepArgs, "tah_topk_mix_args": _capi.TopkMixArgs,
             "tah_kv_append_args": _capi.KvAppendArgs, "tah_additive_mask": _capi.AdditiveMask,
             "tah_greedy_step_args": _capi.GreedyStepArgs, "tah_linear_rows_args": _capi.LinearRowsArgs,
             "tah_step_begin_args": _capi.StepBeginArgs, "tah_decider_tail_args": _capi.DeciderTailArgs,
             "tah_greedy_tick_args": _capi.GreedyTickArgs, "tah_sample_rows_args": _capi.SampleRowsArgs,
             "tah_qk_prep_bwd_args": _capi.QkPrepBwdArgs}
    assert ctypes.sizeof(_capi.DuoStream) == 9 * 8 + 8 * 8 + 2 * 4
    if shutil.which("gcc") is None:
        return
    src = tmp_path / "sizes.c"
    src.write_text('#include <stdio.h>\n#include "tah_duo.h"\nint main(void) {\n' +
                   "".join(f'  printf("{n} %zu\\n", sizeof({n}));\n' for n in pairs) + "  return 0;\n}\n")
    exe = tmp_path / "sizes"
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = dict(line.split() for line in subprocess.check_output([str(exe)], text=True).splitlines())
    for n, mirror in pairs.items():
        assert int(got[n]) == ctypes.sizeof(mirror), n


def test_product_ops_refuse_cpu_tensors():
    import pytest
    import torch

    from tah_amd import TahDuoError, ops
    with pytest.raises(TahDuoError):
        ops.hard_index_build(torch.zeros(2, 3, dtype=torch.bool))


def test_argument_checks_run_before_any_device_work():
    """Validation failures are reported from the host side alone: fake (never dereferenced) pointers
    and no GPU are enough to see the error codes for a bad head dimension, a misaligned pointer and a
    row stride beyond what the tile copies can address."""
    from tah_amd import _capi, _lib
    lib = _capi.bind(ctypes.CDLL(_lib.LIB_PATH))

    def args():
        a = _capi.DuoFwdArgs()
        for s in (a.s1,):
            s.q = s.k = s.v = s.o = 0x10000
            s.lse = 0x20000
            s.cu_q = s.cu_k = 0x30000
            s.q_row_stride = s.k_row_stride = s.v_row_stride = s.o_row_stride = 1024
            s.q_head_stride = s.k_head_stride = s.v_head_stride = s.o_head_stride = 128
            s.total_q = s.total_k = 64
        a.nseq, a.hq, a.hkv, a.d, a.scale = 1, 8, 8, 128, 0.1
        return a

    a = args()
    a.d = 64
    assert lib.tah_duo_fwd_varlen(ctypes.byref(a), None) == _capi.TAH_E_SHAPE
    a = args()
    a.hq, a.hkv = 24, 8  # group of 3 query heads per kv head
    assert lib.tah_duo_fwd_varlen(ctypes.byref(a), None) == _capi.TAH_E_SHAPE
    a = args()
    a.s1.k = 0x10008
    assert lib.tah_duo_fwd_varlen(ctypes.byref(a), None) == _capi.TAH_E_ALIGN
    a = args()
    a.s1.q = None
    assert lib.tah_duo_fwd_varlen(ctypes.byref(a), None) == _capi.TAH_E_NULL
    a = args()
    a.s1.k_row_stride = 1 << 23  # rows further apart than the 24-bit multiply of the tile copies covers
    assert lib.tah_duo_fwd_varlen(ctypes.byref(a), None) == _capi.TAH_E_SHAPE
    b = _capi.DuoBwdArgs()
    b.fwd = args()
    b.fwd.s1.v_row_stride = 1 << 23
    for g in (b.g1,):
        g.d_o = g.dq = g.dk = g.dv = 0x40000
        g.delta = 0x50000
        g.do_row_stride = g.dq_row_stride = g.dk_row_stride = g.dv_row_stride = 1024
        g.do_head_stride = g.dq_head_stride = g.dk_head_stride = g.dv_head_stride = 128
    assert lib.tah_duo_bwd_varlen(ctypes.byref(b), None) == _capi.TAH_E_SHAPE
    # the dS workspace: refused when misaligned or smaller than the size function says (before any launch)
    b.fwd.s1.v_row_stride = 1024
    b.fwd.s2.cu_q = b.fwd.s2.cu_k = 0x30000
    need = lib.tah_duo_bwd_workspace_bytes(1, 8, 8, 64, 64, 0, 0, 0, 0)
    assert need == 2 * 8 * 1 * 16384  # (64 / 64 + 1) query slots x 8 heads x one 128-key slot x 16 KiB
    assert lib.tah_duo_bwd_workspace_bytes(1, 8, 8, 64, 4096, 0, 0, 300, 0) == 2 * 8 * 3 * 16384  # bounded by max_seqlen_k
    assert lib.tah_duo_bwd_workspace_bytes(1, 8, 1, 64, 64, 0, 0, 0, 0) == 0                         # 8 query heads per kv head
    b.ds_workspace, b.ds_workspace_bytes = 0x60008, need
    assert lib.tah_duo_bwd_varlen(ctypes.byref(b), None) == _capi.TAH_E_ALIGN
    b.ds_workspace, b.ds_workspace_bytes = 0x60000, need - 1
    assert lib.tah_duo_bwd_varlen(ctypes.byref(b), None) == _capi.TAH_E_WORKSPACE


def test_topk_mix_argument_checks():
    """tah_topk_mix with its optional outputs: what has to be there, in which shape, before anything is launched."""
    from tah_amd import _capi, _lib
    lib = _capi.bind(ctypes.CDLL(_lib.LIB_PATH))

    def args(**kw):
        a = _capi.TopkMixArgs()
        a.logits, a.embedding, a.out = 0x10000, 0x20000, 0x30000
        a.logits_row_stride, a.embedding_row_stride, a.out_row_stride = 4096, 64, 64
        a.rows, a.vocab, a.hidden, a.topk = 2, 4096, 64, 100
        for k, v in kw.items():
            setattr(a, k, v)
        return a

    call = lambda a: lib.tah_topk_mix(ctypes.byref(a), None)
    assert call(args(topk=257)) == _capi.TAH_E_SHAPE                                       # more places than the kernel holds
    assert call(args(out=0)) == _capi.TAH_E_NULL                                           # neither the mix nor the values
    assert call(args(out=0, indices_out=0x50000)) == _capi.TAH_E_NULL                      # indices without values
    assert call(args(values_out=0x40000, values_row_stride=99)) == _capi.TAH_E_SHAPE       # rows of values would overlap
    assert call(args(values_out=0x40001, values_row_stride=100)) == _capi.TAH_E_ALIGN
    assert call(args(values_out=0x40000, values_row_stride=100, indices_out=0x50002)) == _capi.TAH_E_ALIGN
    assert call(args(out=0, values_out=0x40000, values_row_stride=100, out_packed=0x60000)) == _capi.TAH_E_SHAPE  # packed rows need the mix
    assert call(args(rows=0)) == _capi.TAH_OK

