"""Torch-facing operators: thin Python names over the PyTorch-ROCm extension (``tah_amd._C``), which checks the
tensors, allocates outputs through torch, fills the C argument structs of include/tah_duo.h and calls
libtah_duo.so on torch's current HIP stream.  Nothing is computed in Python or by torch operators.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _capi, _lib


def _call(name: str, *args):
    try:
        return getattr(_lib.lib(), name)(*args)
    except RuntimeError as e:  # argument checks and TAH_E_* codes surface as the package's own error type
        if isinstance(e, _capi.TahDuoError):
            raise
        raise _capi.TahDuoError(str(e).split("\nException raised from")[0]) from None


MAX_SCHEDULE_SEQS = 4095


def duo_schedule(cu_q1, cu_k1, cu_q2, cu_k2, pos_q2, hq: int, hkv: int, total_q1: int, total_k1: int, total_k2: int):
    """Launch-order table for the varlen calls over these boundaries: every tile of both depths, heaviest first.

    Built on the device from the boundary tensors (no read-back); pass it as ``schedule=`` to :func:`duo_fwd_varlen` /
    :func:`duo_bwd_varlen` for as long as the boundaries, ``pos_q2`` and the row counts stay the same -- one table
    serves every layer and the backward pass of a batch.  It only changes the order in which tiles are started.
    Returns ``None`` for a single sequence (its tiles are already in that order) or more than 4095 sequences.
    """
    nseq = cu_q1.numel() - 1
    if nseq <= 1 or nseq > MAX_SCHEDULE_SEQS:
        return None
    return _call("duo_schedule", cu_q1, cu_k1, cu_q2, cu_k2, pos_q2, int(hq), int(hkv), int(total_q1), int(total_k1), int(total_k2))


def duo_fwd_varlen(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale: float, schedule=None
                   ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Duo-causal attention forward on packed varlen bf16 tensors.

    q1 [T1q,Hq,D], k1/v1 [T1k,Hkv,D], cu_q1/cu_k1 int32 [nseq+1]: depth-0 stream.
    q2 [T2q,Hq,D], k2/v2 [T2k,Hkv,D], pos_q2/pos_k2 int32, cu_q2/cu_k2: depth-1 stream
    (hard tokens).  ``schedule``: table from :func:`duo_schedule` or None.  Returns o1, lse1 [Hq,T1q], o2, lse2 [Hq,T2q].
    """
    return _call("duo_fwd_varlen", q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, float(scale), schedule)


# The backward pass can hand dS from the dK/dV kernel to the dQ kernel through a workspace instead of computing the
# scores twice (``tah_duo_bwd_varlen`` with ``ds_workspace``): 5 matrix products per tile pair instead of 7.  The
# workspace holds about total_q * max_seqlen_k * Hq * 2 bytes; calls that would need more than DS_EXCHANGE_MAX_BYTES
# (or Hq / Hkv > 4) run the three-kernel backward.  One buffer per device is kept and grown on demand: the calls of
# a backward pass run one after another on one stream and nothing in it outlives a call.
DS_EXCHANGE = True
DS_EXCHANGE_MAX_BYTES = 24 << 30
_ds_workspaces = {}


def duo_bwd_workspace_bytes(nseq: int, hq: int, hkv: int, total_q1: int, total_k1: int, total_q2: int, total_k2: int,
                            max_seqlen_k1: int = 0, max_seqlen_k2: int = 0) -> int:
    """Bytes of ``ds_workspace`` for a backward call of these sizes (0: the call cannot use one)."""
    return int(_call("duo_bwd_workspace_bytes", int(nseq), int(hq), int(hkv), int(total_q1), int(total_k1), int(total_q2),
                     int(total_k2), int(max_seqlen_k1), int(max_seqlen_k2)))


def _ds_workspace(device, nbytes: int):
    buf = _ds_workspaces.get(device)
    if buf is None or buf.numel() < nbytes:
        _ds_workspaces[device] = None  # release the old one before the larger one is requested
        buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _ds_workspaces[device] = buf
    return buf


def duo_bwd_varlen(q1, k1, v1, o1, lse1, do1, cu_q1, cu_k1, q2, k2, v2, o2, lse2, do2, pos_q2, pos_k2, cu_q2, cu_k2,
                   scale: float, schedule=None, ds_workspace=None, max_seqlen_k1: int = 0, max_seqlen_k2: int = 0):
    """Backward of :func:`duo_fwd_varlen`; returns dq1, dk1, dv1, dq2, dk2, dv2 (bf16).

    ``ds_workspace``: a uint8 tensor of at least :func:`duo_bwd_workspace_bytes` bytes, ``False`` for the three-kernel
    backward, or None: the package's own buffer when ``DS_EXCHANGE`` is on and the call fits ``DS_EXCHANGE_MAX_BYTES``.
    ``max_seqlen_k1`` / ``max_seqlen_k2``: upper bounds on one sequence's key rows per depth (0: unknown); they only
    make the workspace smaller.
    """
    if ds_workspace is None and DS_EXCHANGE:
        need = duo_bwd_workspace_bytes(cu_q1.numel() - 1, q1.shape[1], k1.shape[1], q1.shape[0], k1.shape[0], q2.shape[0],
                                       k2.shape[0], max_seqlen_k1, max_seqlen_k2)
        if 0 < need <= DS_EXCHANGE_MAX_BYTES:
            ds_workspace = _ds_workspace(q1.device, need)
    if ds_workspace is False:
        ds_workspace = None
    return tuple(_call("duo_bwd_varlen", q1, k1, v1, o1, lse1, do1, cu_q1, cu_k1, q2, k2, v2, o2, lse2, do2, pos_q2, pos_k2,
                       cu_q2, cu_k2, float(scale), schedule, ds_workspace, int(max_seqlen_k1), int(max_seqlen_k2)))


def duo_fwd_masked(q, k, v, mask, nseq: int, scale: float):
    """Compatibility mode: ``softmax(q k^T * scale + mask) v`` with a dense additive mask.

    q [B*Tq,Hq,D], k/v [B*Tkv,Hkv,D] (batch rows one after another), mask (B|1, Hq|1, Tq, Tkv).
    Returns o [B*Tq,Hq,D] and lse [Hq, B*Tq].
    """
    return _call("duo_fwd_masked", q, k, v, mask, int(nseq), float(scale))


def duo_bwd_masked(q, k, v, o, lse, d_o, mask, nseq: int, scale: float):
    """Backward of :func:`duo_fwd_masked`; returns dq, dk, dv (bf16)."""
    return tuple(_call("duo_bwd_masked", q, k, v, o, lse, d_o, mask, int(nseq), float(scale)))


def hard_index_build(mask: torch.Tensor):
    """(B, S) bool/uint8 mask -> pos int32 [B*S cap], flat int32, seq int32, cu int32 [B+1].

    Only the first cu[B] entries of pos/flat/seq are defined.  No host sync.
    """
    return _call("hard_index_build", mask)


def pad_rows_build(cu: torch.Tensor, seq_of: torch.Tensor, n: int, width: int, n_dev: Optional[torch.Tensor] = None,
                   overflow: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of the packed entries inside the right-padded (B, width) layout.  ``n_dev`` (device int32, one
    element): only the first ``min(n, n_dev)`` entries are defined -- ``n`` may then be an upper bound."""
    return _call("pad_rows_build", cu, seq_of, int(n), int(width), n_dev, overflow)


def rows_copy(src: torch.Tensor, src_rows: Optional[torch.Tensor], dst: torch.Tensor,
              dst_rows: Optional[torch.Tensor], n: int, dst_enable: Optional[torch.Tensor] = None,
              n_dev: Optional[torch.Tensor] = None) -> None:
    """dst[dst_rows[r]] = src[src_rows[r]] for r < n; src/dst are [rows, ...] with contiguous rows.

    dst_enable (bool/uint8, one entry per row of dst): rows whose entry is 0 are left untouched.
    n_dev (device int32, one element): entries r >= n_dev are skipped too, so ``n`` may be an upper bound
    and the true count never has to reach the host.
    """
    _call("rows_copy", src, src_rows, dst, dst_rows, int(n), dst_enable, n_dev)


def topk_mix(logits: torch.Tensor, embedding: torch.Tensor, topk: int, row_enable: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None, out_packed: Optional[torch.Tensor] = None,
             zero_disabled: bool = False, values_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Soft input embedding of hard tokens (tah_model.py:57-75): logits bf16 [rows, V] -> bf16 [rows, H], the
    softmax over each row's top-k logits times the matching rows of ``embedding`` [V, H].  ``row_enable``
    (bool/uint8 [rows]): rows with 0 are skipped and keep what ``out`` held (zeros when ``out`` is not given, or with
    ``zero_disabled``).  ``out_packed`` (bf16 [32 * H], rows <= 32) also receives the rows as the rows operand of
    ``linear_rows``.  ``values_out`` (bf16 [rows, min(topk, V)]) also receives the top-k logits themselves, largest
    first, as ``torch.topk(logits, topk).values`` holds them."""
    return _call("topk_mix", logits, embedding, int(topk), row_enable, out, out_packed, bool(zero_disabled), values_out)


def topk_values(logits: torch.Tensor, topk: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``torch.topk(logits, min(topk, V), dim=-1).values`` for bf16 logits [rows, V] (``tah_topk_mix`` producing only
    its ``values_out``): the logit features of the iteration decider (tah/model/iter_decider.py:281).  ``out``: a bf16
    [rows, W >= k] matrix whose first k columns take the values (the rest is left as it is)."""
    return _call("topk_values", logits, int(topk), None, out)


def topk(logits: torch.Tensor, k: int):
    """``(values, indices)`` of the k largest entries of every row of bf16 logits [rows, V], largest first, equal values by
    ascending index (``torch.topk`` leaves the order and the choice among equal values open): values bf16, indices int32.
    k <= 256."""
    idx = torch.empty(logits.size(0), min(int(k), logits.size(1)), dtype=torch.int32, device=logits.device)
    return _call("topk_values", logits, int(k), idx, None), idx


def sample_rows(logits: torch.Tensor, uniforms: torch.Tensor, temperature: float, *, top_p: float = 1.0, min_p: float = 0.0,
                logits_prev: Optional[torch.Tensor] = None, add_prev: Optional[torch.Tensor] = None,
                row_enable: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of bf16 logits [rows, V] by temperature sampling with the min_p and top_p filters of
    ``sample_next_token`` (tah/model/utils.py:84-125, ``top_k == 0``), in one launch and without a sort over the vocabulary
    (``tah_sample_rows``).  ``uniforms`` float32 [rows] in [0, 1): the row's random number (``torch.rand``); the draw is the
    inverse-CDF draw over the tokens in descending order of probability, equal ones by ascending index.  Rows whose
    ``add_prev`` entry (int32 [rows]) is not 0 draw from ``logits_prev + logits`` (summed in bf16).  Returns int64 [rows]."""
    if out is None:
        out = torch.zeros(logits.size(0), dtype=torch.int64, device=logits.device)
    _call("sample_rows", logits, logits_prev, add_prev, uniforms, out, None, row_enable, float(temperature), float(top_p), float(min_p))
    return out


def sample_probs(logits: torch.Tensor, temperature: float, *, top_p: float = 1.0, min_p: float = 0.0,
                 logits_prev: Optional[torch.Tensor] = None, add_prev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The distribution :func:`sample_rows` draws from, float32 [rows, V]: softmax(logits / temperature), then min_p and
    top_p, each renormalised; zero outside the filters."""
    probs = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
    _call("sample_rows", logits, logits_prev, add_prev, None, None, probs, None, float(temperature), float(top_p), float(min_p))
    return probs


def silu_mul(gate_up: torch.Tensor, norm_input: Optional[torch.Tensor] = None, norm_eps: float = 0.0) -> torch.Tensor:
    """``silu(gate) * up`` of a fused gate|up projection, bf16 [rows, 2*I] -> [rows, I], in one launch.

    ``norm_input`` [rows, hidden] folds the MLP's input RMSNorm in: ``gate_up`` is then the projection of these
    un-normalised rows through a weight that carries the norm's weight, and gate and up are multiplied by the row's
    ``rsqrt(mean(norm_input**2) + norm_eps)`` first."""
    return _call("silu_mul", gate_up, norm_input, float(norm_eps))


def step_begin(tok, pos, finished, embed, cos_table, sin_table, *, x, x_packed, cos_rows, sin_rows, slot, q_pos, active,
               phase=None, x_alt=None, hard_len=None, q_depth=None, append_at=None, eligible=None) -> None:
    """Start of a generation step in one launch (``tah_step_begin``), results written into the keyword tensors: per
    row ``active = ~finished``; ``slot`` = row index and ``q_pos`` = ``pos`` for active rows, -1 otherwise; the rotary
    rows of ``pos`` (clamped into the tables) in ``cos_rows`` / ``sin_rows`` [rows, 128]; the embedding row of ``tok`` in
    ``x`` [rows, H] and, when given, in ``x_packed`` [32 * H] (the rows operand of ``linear_rows``).

    For a batch whose rows are at different latent iterations (``greedy_tick``): ``phase`` (int32 [rows]) != 0 marks rows at
    their second iteration, whose input is ``x_alt[row]`` instead of the embedding row; ``q_depth`` receives the phase,
    ``append_at`` ``hard_len`` for such rows and ``pos`` for the others, ``eligible`` active rows at their first iteration."""
    _call("step_begin", tok, pos, finished, embed, cos_table, sin_table, x, x_packed, cos_rows, sin_rows, slot, q_pos, active,
          phase, x_alt, hard_len, q_depth, append_at, eligible)


def greedy_tick(logits, logits_prev, eos: int, limit: int, *, hard_now, phase, tok, finished, pos, out_tokens, out_len, hard_len,
                n_hard, n_steps, chosen=None) -> None:
    """End of a tick in which every row advanced by one latent iteration of its own token (``tah_greedy_tick``), all
    updates in place: rows at phase 0 with ``hard_now`` move to phase 1; every other unfinished row gets its token (arg-max
    of ``logits``, or of ``bf16(logits_prev + logits)`` at phase 1) in ``out_tokens[row, out_len[row]]`` and the loop's
    bookkeeping; a row is finished at its end-of-sequence token or with ``limit`` tokens.  ``chosen`` (int64 [rows]):
    tokens to take instead of the arg-max (sampled from the same final logits by the caller)."""
    _call("greedy_tick", logits, logits_prev, int(eos), int(limit), hard_now, phase, tok, finished, pos, out_tokens, out_len,
          hard_len, n_hard, n_steps, chosen)


def decider_tail(hidden, w2, b2, threshold: float, *, hard, active=None, pos=None, hard_i32=None, slot=None, q_pos=None) -> None:
    """Second layer of a two-layer decider and the decision (``tah_decider_tail``): ``hard = sigmoid(hidden @ w2 + b2) >
    threshold`` (``& active``), with the eager bf16 roundings, written into ``hard`` (bool [rows]); optionally
    ``hard_i32`` (0/1), ``slot`` (row index or -1) and ``q_pos`` (``pos`` or -1) for the second latent iteration."""
    _call("decider_tail", hidden, w2, b2, float(threshold), active, pos, hard, hard_i32, slot, q_pos)


LINEAR_MAX_ROWS = 32


def linear_pack_weight(w: torch.Tensor, gate_up: bool = False) -> torch.Tensor:
    """A linear layer's weight, bf16 [N, K] (``gate_up``: [2N, K], gate rows then up rows), in the order
    ``linear_rows`` streams it (``tah_linear_pack_weight``): flat bf16 of the same number of elements.  Done once per
    weight.  K % 32 == 0, N % 16 == 0 (gate|up: N % 24 == 0 or N % 16 == 0)."""
    return _call("linear_pack_weight", w, bool(gate_up))


def linear_pack_rows(x: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of a decode step, bf16 [rows <= 32, K], as the rows operand of ``linear_rows``: flat bf16 [32 * K], rows
    past the last one zero (``tah_linear_pack_rows``)."""
    return _call("linear_pack_rows", x, out)


def linear_rows(w_packed: torch.Tensor, x_packed: torch.Tensor, rows: int, n: int, k: int, *, gate_up: bool = False,
                residual: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                out_packed: Optional[torch.Tensor] = None, want_out: bool = True, norm_eps: Optional[float] = None,
                bias: Optional[torch.Tensor] = None, relu: bool = False, gelu: bool = False,
                ln_colsum: Optional[torch.Tensor] = None):
    """A linear layer of a decode step on packed operands (``tah_linear_rows``), bf16, rows <= 32.

    ``x @ w.T`` [rows, N], plus ``residual`` [rows, N] when given (``out=residual`` updates it in place); with
    ``gate_up``, ``silu(x @ gate.T) * (x @ up.T)``.  With ``norm_eps`` the products are first multiplied by the row's
    ``rsqrt(mean(x**2) + norm_eps)``: an RMSNorm of the rows whose weight sits in w (the MLP's input norm for gate|up,
    the final norm for an output head).  ``bias`` [N] is added to the rounded product and ``relu`` or ``gelu`` (the exact
    one) applied last (the first layer of a small MLP; not with ``gate_up``).  With ``ln_colsum`` (float32 [N], the sums of
    the weight's rows) ``norm_eps`` is a LayerNorm's: the product becomes ``(x @ w.T - mean(x) * ln_colsum) * rsqrt(var(x) +
    norm_eps)``, a layer behind a LayerNorm whose scale sits in w and whose shift sits in ``bias``.  ``out_packed`` [32 * N] also
    receives the result as the next layer's rows operand; ``want_out=False`` with ``out_packed`` writes only that.
    Returns the row-major result (None when it was not asked for)."""
    if relu and gelu:
        raise ValueError("linear_rows: one activation")
    norm = 0 if norm_eps is None else (2 if ln_colsum is not None else 1)
    if ln_colsum is not None and norm_eps is None:
        raise ValueError("linear_rows: ln_colsum needs the LayerNorm's eps")
    return _call("linear_rows", w_packed, x_packed, int(rows), int(n), int(k), bool(gate_up), residual, out, out_packed,
                 bool(want_out), norm, float(norm_eps or 0.0), bias, 1 if relu else (2 if gelu else 0), ln_colsum)


def greedy_step(logits0, logits1, hard, eos: int, tok, finished, pos, out_tokens, step_idx, out_len, n_hard, n_steps) -> None:
    """One greedy generation step after the logits (``tah_greedy_step``), all updates in place on the device.

    Per row: final logits = ``logits0`` (bf16 [rows, vocab]), or ``bf16(logits0 + logits1)`` where ``hard`` (bool
    [rows]) is set; ``tok`` = their arg-max (0 for finished rows); a row whose token is ``eos`` (>= 0) becomes
    ``finished`` and the token stays out of its output; ``out_tokens[:, step_idx]`` and ``out_len`` record the
    output, ``pos`` advances for the rows that decoded, ``n_steps`` / ``n_hard`` count them.
    """
    _call("greedy_step", logits0, logits1, hard, int(eos), tok, finished, pos, out_tokens, step_idx, out_len, n_hard, n_steps)
