"""ctypes mirror of include/tah_duo.h: structs, prototypes, error codes.

The package itself reaches the library through its PyTorch extension (``tah_amd._C``, csrc/torch_ext.cpp).
This module describes the same C ABI for callers that want to bind it without torch (``bind`` attaches the
prototypes to a ``ctypes.CDLL``) and for the tests that call entry points with hand-made arguments.
"""
from __future__ import annotations

import ctypes as C

ABI_VERSION = 7

c_void_p, c_int32, c_int64, c_float = C.c_void_p, C.c_int32, C.c_int64, C.c_float


# error codes of include/tah_duo.h
TAH_OK, TAH_E_NULL, TAH_E_SHAPE, TAH_E_ALIGN, TAH_E_LAUNCH, TAH_E_WORKSPACE, TAH_E_SCRATCH = 0, -1, -2, -3, -4, -5, -6
STATIC_SCRATCH_BYTES = 16 << 20


class DuoStream(C.Structure):
    """``tah_duo_stream``"""

    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("o", c_void_p), ("lse", c_void_p),
        ("cu_q", c_void_p), ("cu_k", c_void_p), ("pos_q", c_void_p), ("pos_k", c_void_p),
        ("q_row_stride", c_int64), ("q_head_stride", c_int64),
        ("k_row_stride", c_int64), ("k_head_stride", c_int64),
        ("v_row_stride", c_int64), ("v_head_stride", c_int64),
        ("o_row_stride", c_int64), ("o_head_stride", c_int64),
        ("total_q", c_int32), ("total_k", c_int32),
    ]


class DuoFwdArgs(C.Structure):
    """``tah_duo_fwd_args``"""

    _fields_ = [
        ("s1", DuoStream), ("s2", DuoStream),
        ("nseq", c_int32), ("hq", c_int32), ("hkv", c_int32), ("d", c_int32),
        ("scale", c_float),
        ("schedule", c_void_p),
    ]


class DuoScheduleArgs(C.Structure):
    """``tah_duo_schedule_args``"""

    _fields_ = [
        ("cu_q1", c_void_p), ("cu_k1", c_void_p), ("cu_q2", c_void_p), ("cu_k2", c_void_p), ("pos_q2", c_void_p),
        ("nseq", c_int32), ("hq", c_int32), ("hkv", c_int32),
        ("total_q1", c_int32), ("total_k1", c_int32), ("total_q2", c_int32), ("total_k2", c_int32),
        ("schedule", c_void_p), ("schedule_bytes", C.c_size_t),
    ]


class DuoBwdStream(C.Structure):
    """``tah_duo_bwd_stream``"""

    _fields_ = [
        ("d_o", c_void_p), ("dq", c_void_p), ("dk", c_void_p), ("dv", c_void_p), ("delta", c_void_p),
        ("do_row_stride", c_int64), ("do_head_stride", c_int64),
        ("dq_row_stride", c_int64), ("dq_head_stride", c_int64),
        ("dk_row_stride", c_int64), ("dk_head_stride", c_int64),
        ("dv_row_stride", c_int64), ("dv_head_stride", c_int64),
    ]


class DuoBwdArgs(C.Structure):
    """``tah_duo_bwd_args``"""

    _fields_ = [("fwd", DuoFwdArgs), ("g1", DuoBwdStream), ("g2", DuoBwdStream),
                ("ds_workspace", c_void_p), ("ds_workspace_bytes", C.c_size_t),
                ("max_seqlen_k1", c_int32), ("max_seqlen_k2", c_int32)]


class AdditiveMask(C.Structure):
    """``tah_additive_mask``"""

    _fields_ = [
        ("mask", c_void_p),
        ("seq_stride", c_int64), ("head_stride", c_int64), ("q_stride", c_int64), ("k_stride", c_int64),
        ("dtype", c_int32),
    ]


class KvSegment(C.Structure):
    """``tah_kv_segment``"""

    _fields_ = [
        ("k", c_void_p), ("v", c_void_p), ("pos", c_void_p), ("start", c_void_p), ("len", c_void_p),
        ("k_row_stride", c_int64), ("k_head_stride", c_int64), ("v_row_stride", c_int64), ("v_head_stride", c_int64),
        ("capacity", c_int32), ("nslots", c_int32),
    ]


class DuoDecodeArgs(C.Structure):
    """``tah_duo_decode_args``"""

    _fields_ = [
        ("q", c_void_p), ("o", c_void_p), ("lse", c_void_p),
        ("q_row_stride", c_int64), ("q_head_stride", c_int64), ("o_row_stride", c_int64), ("o_head_stride", c_int64),
        ("q_slot", c_void_p), ("q_pos", c_void_p), ("q_depth", c_void_p),
        ("depth", c_int32),
        ("c1", KvSegment), ("c2", KvSegment),
        ("workspace", c_void_p), ("workspace_bytes", C.c_size_t),
        ("nq", c_int32), ("hq", c_int32), ("hkv", c_int32), ("d", c_int32),
        ("scale", c_float),
        ("o_packed", c_void_p),
    ]


class LinearRowsArgs(C.Structure):
    """``tah_linear_rows_args``"""

    _fields_ = [
        ("w_packed", c_void_p), ("x_packed", c_void_p), ("residual", c_void_p), ("out", c_void_p), ("out_packed", c_void_p),
        ("residual_row_stride", c_int64), ("out_row_stride", c_int64),
        ("rows", c_int32), ("n", c_int32), ("k", c_int32), ("kind", c_int32), ("input_norm", c_int32), ("norm_eps", c_float),
        ("bias", c_void_p), ("activation", c_int32), ("ln_colsum", c_void_p),
    ]


class StepBeginArgs(C.Structure):
    """``tah_step_begin_args``"""

    _fields_ = [
        ("tok", c_void_p), ("pos", c_void_p), ("finished", c_void_p), ("embed", c_void_p), ("embed_row_stride", c_int64),
        ("cos_table", c_void_p), ("sin_table", c_void_p),
        ("rows", c_int32), ("vocab", c_int32), ("hidden", c_int32), ("table_rows", c_int32),
        ("x", c_void_p), ("x_row_stride", c_int64), ("x_packed", c_void_p), ("cos_rows", c_void_p), ("sin_rows", c_void_p),
        ("slot", c_void_p), ("q_pos", c_void_p), ("active", c_void_p),
        ("phase", c_void_p), ("x_alt", c_void_p), ("x_alt_row_stride", c_int64), ("hard_len", c_void_p),
        ("q_depth", c_void_p), ("append_at", c_void_p), ("eligible", c_void_p),
    ]


class GreedyTickArgs(C.Structure):
    """``tah_greedy_tick_args``"""

    _fields_ = [
        ("logits", c_void_p), ("logits_prev", c_void_p), ("row_stride", c_int64), ("row_stride_prev", c_int64),
        ("rows", c_int32), ("vocab", c_int32), ("eos", c_int32), ("limit", c_int32),
        ("hard_now", c_void_p), ("phase", c_void_p), ("tok", c_void_p), ("finished", c_void_p), ("pos", c_void_p),
        ("out_tokens", c_void_p), ("out_stride", c_int64), ("out_len", c_void_p), ("hard_len", c_void_p),
        ("n_hard", c_void_p), ("n_steps", c_void_p), ("chosen", c_void_p),
    ]


class DeciderTailArgs(C.Structure):
    """``tah_decider_tail_args``"""

    _fields_ = [
        ("hidden", c_void_p), ("hidden_row_stride", c_int64), ("w2", c_void_p), ("b2", c_void_p), ("threshold", c_float),
        ("rows", c_int32), ("width", c_int32), ("active", c_void_p), ("pos", c_void_p), ("hard", c_void_p),
        ("hard_i32", c_void_p), ("slot", c_void_p), ("q_pos", c_void_p),
    ]


LINEAR_PLAIN, LINEAR_GATE_UP = 0, 1
LINEAR_MAX_ROWS = 32


class KvAppendArgs(C.Structure):
    """``tah_kv_append_args``"""

    _fields_ = [
        ("k_new", c_void_p), ("v_new", c_void_p), ("pos_new", c_void_p),
        ("k_row_stride", c_int64), ("k_head_stride", c_int64), ("v_row_stride", c_int64), ("v_head_stride", c_int64),
        ("cu_new", c_void_p), ("slot_of", c_void_p),
        ("nseq", c_int32), ("total_new", c_int32), ("hkv", c_int32), ("d", c_int32),
        ("cache", KvSegment),
        ("overflow", c_void_p),
    ]


class QkPrepArgs(C.Structure):
    """``tah_qk_prep_args``"""

    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("q_out", c_void_p), ("k_out", c_void_p), ("v_out", c_void_p),
        ("q_row_stride", c_int64), ("q_head_stride", c_int64), ("k_row_stride", c_int64), ("k_head_stride", c_int64),
        ("v_row_stride", c_int64), ("v_head_stride", c_int64),
        ("q_out_row_stride", c_int64), ("q_out_head_stride", c_int64), ("k_out_row_stride", c_int64),
        ("k_out_head_stride", c_int64), ("v_out_row_stride", c_int64), ("v_out_head_stride", c_int64),
        ("q_weight", c_void_p), ("k_weight", c_void_p), ("cos", c_void_p), ("sin", c_void_p),
        ("cos_sin_row_stride", c_int64),
        ("eps", C.c_float),
        ("rows", c_int32), ("hq", c_int32), ("hkv", c_int32), ("d", c_int32),
        ("append", c_int32),
        ("cu_new", c_void_p), ("slot_of", c_void_p), ("pos_new", c_void_p),
        ("nseq", c_int32),
        ("cache", KvSegment),
        ("overflow", c_void_p),
        ("append_one_row_per_seq", c_int32),
        ("norm_input", c_void_p), ("norm_input_row_stride", c_int64), ("norm_cols", c_int32), ("norm_eps", C.c_float),
    ]


class GreedyStepArgs(C.Structure):
    """``tah_greedy_step_args``"""

    _fields_ = [
        ("logits0", c_void_p), ("logits1", c_void_p), ("hard", c_void_p),
        ("row_stride0", c_int64), ("row_stride1", c_int64),
        ("rows", c_int32), ("vocab", c_int32), ("eos", c_int32),
        ("tok", c_void_p), ("finished", c_void_p), ("pos", c_void_p), ("out_tokens", c_void_p), ("out_stride", c_int64),
        ("step_idx", c_void_p), ("out_cols", c_int32), ("out_len", c_void_p), ("n_hard", c_void_p), ("n_steps", c_void_p),
    ]


class TopkMixArgs(C.Structure):
    """``tah_topk_mix_args``"""

    _fields_ = [
        ("logits", c_void_p), ("embedding", c_void_p), ("out", c_void_p), ("row_enable", c_void_p),
        ("logits_row_stride", c_int64), ("embedding_row_stride", c_int64), ("out_row_stride", c_int64),
        ("rows", c_int32), ("vocab", c_int32), ("hidden", c_int32), ("topk", c_int32),
        ("out_packed", c_void_p), ("zero_disabled", c_int32),
        ("values_out", c_void_p), ("values_row_stride", c_int64), ("indices_out", c_void_p),
    ]


class SampleRowsArgs(C.Structure):
    """``tah_sample_rows_args``"""

    _fields_ = [
        ("logits", c_void_p), ("logits_prev", c_void_p), ("add_prev", c_void_p), ("row_enable", c_void_p), ("uniforms", c_void_p),
        ("tokens", c_void_p), ("probs", c_void_p),
        ("logits_row_stride", c_int64), ("prev_row_stride", c_int64), ("probs_row_stride", c_int64),
        ("rows", c_int32), ("vocab", c_int32), ("temperature", c_float), ("top_p", c_float), ("min_p", c_float),
    ]


class QkPrepBwdArgs(C.Structure):
    """``tah_qk_prep_bwd_args``"""

    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("dq_out", c_void_p), ("dk_out", c_void_p), ("dq", c_void_p), ("dk", c_void_p),
        ("q_row_stride", c_int64), ("q_head_stride", c_int64), ("k_row_stride", c_int64), ("k_head_stride", c_int64),
        ("dq_out_row_stride", c_int64), ("dq_out_head_stride", c_int64), ("dk_out_row_stride", c_int64), ("dk_out_head_stride", c_int64),
        ("dq_row_stride", c_int64), ("dq_head_stride", c_int64), ("dk_row_stride", c_int64), ("dk_head_stride", c_int64),
        ("q_weight", c_void_p), ("k_weight", c_void_p), ("cos", c_void_p), ("sin", c_void_p), ("cos_sin_row_stride", c_int64),
        ("eps", c_float), ("rows", c_int32), ("hq", c_int32), ("hkv", c_int32), ("d", c_int32),
        ("dw_partial", c_void_p), ("n_partial", c_int32),
    ]


PROTOTYPES = {
    "tah_duo_abi_version": (C.c_int, []),
    "tah_duo_error_string": (C.c_char_p, [C.c_int]),
    "tah_duo_fwd_varlen": (C.c_int, [C.POINTER(DuoFwdArgs), c_void_p]),
    "tah_duo_bwd_varlen": (C.c_int, [C.POINTER(DuoBwdArgs), c_void_p]),
    "tah_duo_bwd_workspace_bytes": (C.c_size_t, [c_int32] * 9),
    "tah_duo_schedule_bytes": (C.c_size_t, [c_int32] * 7),
    "tah_duo_schedule_build": (C.c_int, [C.POINTER(DuoScheduleArgs), c_void_p]),
    "tah_greedy_step": (C.c_int, [C.POINTER(GreedyStepArgs), c_void_p]),
    "tah_silu_mul_normed": (C.c_int, [c_void_p, c_void_p, c_int32, c_int32, c_int64, c_int64, c_void_p, c_int64, c_int32, c_float,
                                      c_void_p]),
    "tah_duo_fwd_masked": (C.c_int, [C.POINTER(DuoFwdArgs), C.POINTER(AdditiveMask), c_void_p]),
    "tah_duo_bwd_masked": (C.c_int, [C.POINTER(DuoBwdArgs), C.POINTER(AdditiveMask), c_void_p]),
    "tah_duo_decode_workspace_bytes": (C.c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "tah_duo_decode": (C.c_int, [C.POINTER(DuoDecodeArgs), c_void_p]),
    "tah_duo_decode_static": (C.c_int, [C.POINTER(DuoDecodeArgs), c_void_p]),
    "tah_step_begin": (C.c_int, [C.POINTER(StepBeginArgs), c_void_p]),
    "tah_greedy_tick": (C.c_int, [C.POINTER(GreedyTickArgs), c_void_p]),
    "tah_decider_tail": (C.c_int, [C.POINTER(DeciderTailArgs), c_void_p]),
    "tah_linear_pack_weight": (C.c_int, [c_void_p, c_int64, c_void_p, c_int32, c_int32, c_int32, c_void_p]),
    "tah_linear_pack_rows": (C.c_int, [c_void_p, c_int64, c_void_p, c_int32, c_int32, c_void_p]),
    "tah_linear_rows": (C.c_int, [C.POINTER(LinearRowsArgs), c_void_p]),
    "tah_kv_append": (C.c_int, [C.POINTER(KvAppendArgs), c_void_p]),
    "tah_qk_prep": (C.c_int, [C.POINTER(QkPrepArgs), c_void_p]),
    "tah_duo_decode_step": (C.c_int, [C.POINTER(QkPrepArgs), C.POINTER(DuoDecodeArgs), c_void_p, c_void_p, c_void_p]),
    "tah_duo_decode_step_supported": (C.c_int, [c_int32, c_int32, c_int32, c_int32]),
    "tah_topk_mix": (C.c_int, [C.POINTER(TopkMixArgs), c_void_p]),
    "tah_qk_prep_bwd": (C.c_int, [C.POINTER(QkPrepBwdArgs), c_void_p]),
    "tah_sample_rows": (C.c_int, [C.POINTER(SampleRowsArgs), c_void_p]),
    "tah_silu_mul": (C.c_int, [c_void_p, c_void_p, c_int32, c_int32, c_int64, c_int64, c_void_p]),
    "tah_hard_index_build": (C.c_int, [c_void_p, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "tah_pad_rows_build": (C.c_int, [c_void_p, c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_void_p]),
    "tah_rows_copy": (C.c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_int64, c_int64,
                                c_int64, c_void_p]),
}


class TahDuoError(RuntimeError):
    pass


def bind(lib: C.CDLL) -> C.CDLL:
    """Attach prototypes; raises AttributeError if a declared symbol is missing."""
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    got = lib.tah_duo_abi_version()
    if got != ABI_VERSION:
        raise TahDuoError(f"libtah_duo ABI version {got}, expected {ABI_VERSION}")
    return lib


def check(lib: C.CDLL, rc: int, what: str) -> None:
    if rc != 0:
        raise TahDuoError(f"{what}: {lib.tah_duo_error_string(rc).decode()} (code {rc})")
