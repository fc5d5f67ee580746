"""Native per-layer KV storage for the duo-causal decode path.

One :class:`KvSlabs` holds one depth (iteration) of one decoder layer: a slab
of ``capacity`` rows per sequence slot, head-major inside the slab
(``[slot, Hkv, capacity, D]``), so that the decode kernel streams each
(sequence, kv head) as one contiguous run.  Lengths live on the device; appends
and reads never synchronise with the host.  This replaces the growing
``torch.cat`` tensors of the reference cache (tah/model/causal_cache.py:84-95).
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _capi
from .ops import _call


class KvSlabs:
    def __init__(self, nslots: int, capacity: int, hkv: int, d: int = 128, *, with_pos: bool, device, dtype=torch.bfloat16):
        self.nslots, self.capacity, self.hkv, self.d = nslots, capacity, hkv, d
        self.k = torch.zeros((nslots, hkv, capacity, d), dtype=dtype, device=device)
        self.v = torch.zeros((nslots, hkv, capacity, d), dtype=dtype, device=device)
        self.pos = torch.zeros((nslots, capacity), dtype=torch.int32, device=device) if with_pos else None
        # first row of each slab in units of row_stride (= d elements)
        self.start = (torch.arange(nslots, dtype=torch.int64, device=device) * (hkv * capacity)).to(torch.int32)
        self.len = torch.zeros(nslots, dtype=torch.int32, device=device)
        self.overflow = torch.zeros(1, dtype=torch.int32, device=device)
        if nslots * hkv * capacity >= 2 ** 31:
            raise _capi.TahDuoError("KvSlabs: more than 2^31 rows")

    def reorder(self, index: torch.Tensor) -> None:
        """Slot i takes the rows, positions and length of slot index[i] (beam search: several beams may continue
        the same sequence).  In place, through one temporary copy per tensor, so the slab addresses stay valid."""
        idx = index.to(device=self.k.device, dtype=torch.int64)
        if idx.numel() != self.nslots:
            raise _capi.TahDuoError(f"KvSlabs.reorder: {idx.numel()} indices for {self.nslots} slots")
        for t in (self.k, self.v, self.pos, self.len):
            if t is not None:
                t.copy_(t.index_select(0, idx))

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor, cu_new: torch.Tensor,
               pos_new: Optional[torch.Tensor] = None, slot_of: Optional[torch.Tensor] = None) -> None:
        """Append rows [cu_new[i], cu_new[i+1]) of k_new/v_new ([rows, Hkv, D]) to slot slot_of[i] (default i;
        a negative entry skips that sequence's rows)."""
        _call("kv_append", k_new, v_new, cu_new, pos_new, slot_of, self.k, self.v, self.pos, self.start, self.len, self.overflow)


class _QkNormRope(torch.autograd.Function):
    """``tah_qk_prep`` without append, differentiable: backward is one ``tah_qk_prep_bwd`` launch (gradients of q, k and
    of the two norm weights; cos / sin are tables, not parameters)."""

    # workgroups of the backward launch: each walks every BWD_PARTIALS-th row and leaves one row of partial weight
    # gradients, which are added up here in a fixed order
    BWD_PARTIALS = 4096

    @staticmethod
    def forward(ctx, q, k, q_weight, k_weight, cos, sin, eps):
        q_out, k_out = torch.empty_like(q), torch.empty_like(k)
        _call("qk_prep", q, k, None, q_out, k_out, q_weight, k_weight, cos, sin, float(eps), None, None, None, None, None, None,
              None, None, None, False, None, None, 0.0)
        ctx.save_for_backward(q, k, q_weight, k_weight, cos, sin)
        ctx.eps = float(eps)
        return q_out, k_out

    @staticmethod
    def backward(ctx, dq_out, dk_out):
        q, k, q_weight, k_weight, cos, sin = ctx.saved_tensors
        n = max(1, min(_QkNormRope.BWD_PARTIALS, q.shape[0]))
        dq, dk, part = _call("qk_prep_bwd", q, k, dq_out.contiguous(), dk_out.contiguous(), q_weight, k_weight, cos, sin, ctx.eps, n)
        dw = part.sum(0)
        return dq, dk, dw[0].to(q_weight.dtype), dw[1].to(k_weight.dtype), None, None, None


def qk_norm_rope(q: torch.Tensor, k: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor,
                 cos: torch.Tensor, sin: torch.Tensor, eps: float, *, v: Optional[torch.Tensor] = None,
                 cache: Optional[KvSlabs] = None, cu_new: Optional[torch.Tensor] = None,
                 pos_new: Optional[torch.Tensor] = None, slot_of: Optional[torch.Tensor] = None,
                 in_place: bool = False, one_row_per_seq: bool = False, norm_input: Optional[torch.Tensor] = None,
                 norm_eps: float = 0.0):
    """Per-head RMSNorm of q and k, rotary embedding of both and, with ``cache``, the KV append, in one
    kernel: the steps of ``Qwen3Attention.forward`` between the projections and the attention call
    (``q_norm``, ``k_norm``, ``apply_rotary_pos_emb``, ``past_key_values.update``), with bf16 roundings
    where the eager modules round.

    q ``[rows, Hq, 128]``, k / v ``[rows, Hkv, 128]`` (token-major, as the projections produce them),
    weights ``[128]``, cos / sin ``[rows, 128]``, all bf16.  Returns ``(q_out, k_out)``; with ``cache``
    K and V go to the slabs (rows ``[cu_new[i], cu_new[i+1])`` to slot ``slot_of[i]``) and ``k_out`` is
    ``None``.  ``one_row_per_seq=True`` (a decode step: every sequence brings at most one row, all slots
    different) lets the same launch advance the slab lengths.

    ``norm_input`` ``[rows, hidden]`` folds the layer's input RMSNorm in: q, k, v are then projections of these
    un-normalised rows through weights that carry the norm's weight, and the kernel multiplies every head by the
    row's ``rsqrt(mean(norm_input**2) + norm_eps)`` first.  Without a cache the scaled V comes back as a third
    result.

    With gradients enabled and q, k or a weight requiring them (training): the plain form only (no cache, no
    ``norm_input``, not in place), differentiable through ``tah_qk_prep_bwd``."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, q_weight, k_weight)):
        if cache is not None or norm_input is not None or in_place:
            raise _capi.TahDuoError("qk_norm_rope: the differentiable form takes neither a cache to append to, nor a folded "
                                    "input norm, nor in_place")
        return _QkNormRope.apply(q, k, q_weight, k_weight, cos, sin, eps)
    q_out = q if in_place else torch.empty_like(q)
    if cache is not None:
        _call("qk_prep", q, k, v, q_out, None, q_weight, k_weight, cos, sin, float(eps), cache.k, cache.v, cache.pos,
              cache.start, cache.len, cache.overflow, cu_new, pos_new, slot_of, bool(one_row_per_seq), None, norm_input,
              float(norm_eps))
        return q_out, None
    k_out = k if in_place else torch.empty_like(k)
    v_out = None
    if norm_input is not None and v is not None:
        v_out = v if in_place else torch.empty_like(v)
    _call("qk_prep", q, k, v, q_out, k_out, q_weight, k_weight, cos, sin, float(eps), None, None, None, None, None, None,
          None, None, None, False, v_out, norm_input, float(norm_eps))
    return (q_out, k_out) if v_out is None else (q_out, k_out, v_out)


_WORKSPACES = {}


def decode_step_supported(nq: int, hq: int, hkv: int, capacity1: int) -> bool:
    """Whether :func:`decode_step` takes a call of these sizes (``tah_duo_decode_step_supported``)."""
    return bool(_call("duo_decode_step_supported", int(nq), int(hq), int(hkv), int(capacity1)))


def decode_step(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor,
                cos: torch.Tensor, sin: torch.Tensor, eps: float, *, cache: KvSlabs, cu_new: torch.Tensor,
                append_at: torch.Tensor, q_slot: torch.Tensor, q_pos: torch.Tensor, c1: KvSlabs, c2: Optional[KvSlabs],
                scale: float, slot_of: Optional[torch.Tensor] = None, pos_new: Optional[torch.Tensor] = None,
                norm_input: Optional[torch.Tensor] = None, norm_eps: float = 0.0, depth: int = 0,
                q_depth: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                out_packed: Optional[torch.Tensor] = None, append_depth: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``qk_norm_rope(..., cache=cache, one_row_per_seq=True)`` followed by ``decode(...)`` in one launch
    (``tah_duo_decode_step``), for a generation step: q ``[B, Hq, 128]``, k / v ``[B, Hkv, 128]`` are the projections
    of one new token per sequence, ``cache`` (``c1`` or ``c2``) receives the prepared K and V, and row i attends as
    query i.  ``append_at`` int32 [B]: the rows sequence i's segment of ``cache`` holds before the call (the caller's
    own copy of ``cache.len``: the kernel cannot read the lengths while it advances them).  Same cache contents and
    lengths as the two calls, bit for bit, and the same outputs up to the last bit of a rare element.  ``append_depth``
    (int32 [B], 0 / 1): per row the segment (``c1`` / ``c2``) its K and V go to, for a batch whose rows are at different
    latent iterations; ``append_at`` then counts that segment's rows.  Only for sizes :func:`decode_step_supported` accepts."""
    if q.dim() != 3:
        raise _capi.TahDuoError("decode_step: q must be [B, Hq, D]")
    need2 = q_depth is not None or depth >= 1
    if need2 and c2 is None:
        raise _capi.TahDuoError("depth-1 queries need the depth-1 cache")
    o = out if out is not None else torch.empty_like(q)
    two = (c2.k, c2.v, c2.pos, c2.start, c2.len) if need2 else (None,) * 5
    _call("duo_decode_step", q, k, v, q_weight, k_weight, cos, sin, float(eps), cache.k, cache.v, cache.pos, cache.start,
          cache.len, cache.overflow, cu_new, pos_new, slot_of, norm_input, float(norm_eps), append_at, append_depth,
          o, None, q_slot, q_pos, q_depth, int(depth), c1.k, c1.v, c1.start, c1.len, *two, float(scale), out_packed)
    return o


def decode(q: torch.Tensor, q_slot: torch.Tensor, q_pos: torch.Tensor, c1: KvSlabs, c2: Optional[KvSlabs], *,
           scale: float, depth: int = 0, q_depth: Optional[torch.Tensor] = None, return_lse: bool = False,
           out: Optional[torch.Tensor] = None, lse_out: Optional[torch.Tensor] = None, static_scratch: bool = False,
           out_packed: Optional[torch.Tensor] = None):
    """One decode step: q [nq, Hq, D] bf16, one row per (sequence, depth) being decoded.

    Row i belongs to cache slot q_slot[i], sits at position q_pos[i], and sees the
    depth-0 rows with index <= q_pos[i] plus, at depth 1, the depth-1 rows with
    pos <= q_pos[i].  ``q_depth`` (int32 [nq]) overrides ``depth`` per row.
    ``out`` / ``lse_out`` take the results when given.  ``static_scratch=True`` calls
    ``tah_duo_decode_static``: the split-K partials go to the buffer the library holds on the GPU, so with
    ``out`` given the call allocates nothing (callers under graph capture); requests beyond
    ``_capi.STATIC_SCRATCH_BYTES`` raise.  ``out_packed`` (bf16 [32 * Hq * D], nq <= 32) also receives the output as the
    rows operand of ``ops.linear_rows`` for the o projection (rows nq .. 31 are not touched).
    """
    if q.dim() != 3:
        raise _capi.TahDuoError("decode: q must be [nq, Hq, D]")
    nq, hq, d = q.shape
    need2 = q_depth is not None or depth >= 1
    if need2 and c2 is None:
        raise _capi.TahDuoError("depth-1 queries need the depth-1 cache")
    o = out if out is not None else torch.empty((nq, hq, d), dtype=q.dtype, device=q.device)
    if o.shape != (nq, hq, d) or o.dtype != q.dtype or o.stride(2) != 1:
        raise _capi.TahDuoError("decode: out must be a [nq, Hq, D] tensor of q's dtype")
    lse = lse_out if lse_out is not None else (torch.empty((nq, hq), dtype=torch.float32, device=q.device) if return_lse else None)
    ws = None
    if not static_scratch:
        nbytes = _call("decode_workspace_bytes", nq, hq, c1.capacity, c2.capacity if need2 else 0)
        key = (q.device, torch.cuda.current_stream(q.device).cuda_stream if q.is_cuda else 0)
        ws = _WORKSPACES.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
            _WORKSPACES[key] = ws
    two = (c2.k, c2.v, c2.pos, c2.start, c2.len) if need2 else (None,) * 5
    _call("duo_decode", q, o, lse, q_slot, q_pos, q_depth, int(depth), c1.k, c1.v, c1.start, c1.len, *two, ws, float(scale),
          out_packed)
    return (o, lse) if return_lse else o
