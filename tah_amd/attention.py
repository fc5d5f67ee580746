"""Duo-causal attention behind the reference's call sites.

Three layers, from the bottom up:

* :func:`duo_attn_varlen` -- differentiable packed-varlen op (forward and
  backward HIP kernels), both iteration streams in one launch;
* :class:`DuoMask` / :func:`build_attention_mask` -- the stand-in for the dense
  additive mask of ``TaHForCausalLM._build_attention_mask``
  (tah/model/tah_model.py:744-791): same arguments, but it returns a small
  carrier of (positions, valid flags, cache, depth) instead of a (B,1,Tq,Tkv)
  tensor, because the kernels evaluate the predicate themselves;
* :func:`duo_attention_forward` -- a Hugging Face attention-interface callable
  (same signature and return convention as ``sdpa_attention_forward``,
  transformers/integrations/sdpa_attention.py:79-166) that takes the carrier in
  the ``attention_mask`` slot.

Contract inherited from the kernels: within each batch row the valid tokens'
positions are their rank among the valid tokens of that sequence (what the
model's forward computes when ``position_ids`` is None, tah_model.py:555-559),
and a depth-1 token's depth-0 key is already in the cache.  Query rows that are
not valid get zeros.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import kv_cache, ops
from ._capi import TahDuoError
from .cache import TaHDuoCache
from .pack import HardIndex


class _DuoAttnVarlen(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q1, k1, v1, q2, k2, v2, cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2, scale, schedule=None,
                max_seqlen_k1=0, max_seqlen_k2=0):
        o1, lse1, o2, lse2 = ops.duo_fwd_varlen(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale,
                                                schedule)
        ctx.save_for_backward(q1, k1, v1, o1, lse1, q2, k2, v2, o2, lse2, cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2)
        ctx.scale = scale
        ctx.schedule = schedule
        ctx.max_k = (int(max_seqlen_k1), int(max_seqlen_k2))
        ctx.mark_non_differentiable(lse1, lse2)
        return o1, o2, lse1, lse2

    @staticmethod
    def backward(ctx, do1, do2, _dl1, _dl2):
        q1, k1, v1, o1, lse1, q2, k2, v2, o2, lse2, cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2 = ctx.saved_tensors
        c = lambda g, like: (torch.zeros_like(like) if g is None else g.contiguous())
        dq1, dk1, dv1, dq2, dk2, dv2 = ops.duo_bwd_varlen(
            q1, k1, v1, o1, lse1, c(do1, o1), cu_q1, cu_k1, q2, k2, v2, o2, lse2, c(do2, o2),
            pos_q2, pos_k2, cu_q2, cu_k2, ctx.scale, ctx.schedule, max_seqlen_k1=ctx.max_k[0], max_seqlen_k2=ctx.max_k[1])
        return dq1, dk1, dv1, dq2, dk2, dv2, None, None, None, None, None, None, None, None, None, None


def duo_attn_varlen(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale: float,
                    return_lse: bool = False, schedule=None, max_seqlen_k1: int = 0, max_seqlen_k2: int = 0):
    """Duo-causal attention on packed varlen bf16 tensors, differentiable.

    Depth-0 stream: q1 [T1q,Hq,D], k1/v1 [T1k,Hkv,D], cu_q1/cu_k1 int32 [nseq+1].
    Depth-1 stream (hard tokens): q2 [T2q,Hq,D], k2/v2 [T2k,Hkv,D], int32 positions
    pos_q2/pos_k2 and cu_q2/cu_k2.  Key (pos_k, depth_k) is visible to query
    (pos_q, depth_q) iff pos_k <= pos_q and depth_k <= depth_q.  ``schedule``: the launch-order table
    :func:`tah_amd.ops.duo_schedule` built for these boundaries (forward and backward use it), or None.
    ``max_seqlen_k1`` / ``max_seqlen_k2``: upper bounds on one sequence's key rows per depth (0: unknown); they only
    make the backward pass's dS workspace smaller (:func:`tah_amd.ops.duo_bwd_varlen`).
    Returns (o1, o2).
    """
    o1, o2, lse1, lse2 = _DuoAttnVarlen.apply(q1, k1, v1, q2, k2, v2, cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2,
                                              float(scale), schedule, max_seqlen_k1, max_seqlen_k2)
    return (o1, o2, lse1, lse2) if return_lse else (o1, o2)


class _AttnMasked(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, mask, nseq, scale):
        o, lse = ops.duo_fwd_masked(q, k, v, mask, nseq, scale)
        ctx.save_for_backward(q, k, v, o, lse, mask)
        ctx.nseq, ctx.scale = nseq, scale
        ctx.mark_non_differentiable(lse)
        return o, lse

    @staticmethod
    def backward(ctx, d_o, _dl):
        q, k, v, o, lse, mask = ctx.saved_tensors
        d_o = torch.zeros_like(o) if d_o is None else d_o.contiguous()
        dq, dk, dv = ops.duo_bwd_masked(q, k, v, o, lse, d_o, mask, ctx.nseq, ctx.scale)
        return dq, dk, dv, None, None, None


def attn_additive_mask(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, mask: torch.Tensor,
                       scale: float, return_lse: bool = False):
    """Compatibility mode: what sdpa_attention_forward computes today (sdpa_attention.py:79-166) --
    ``softmax(q k^T * scale + mask) v`` with GQA by head grouping -- for callers that still pass the dense
    additive mask of tah_model.py:744-791.  query (B,Hq,Tq,D), key/value (B,Hkv,Tkv,D), mask
    (B|1, Hq|1, Tq, Tkv) bf16 or float32.  Returns (B,Tq,Hq,D); differentiable in q, k, v.
    Rows whose keys are all hidden come out as zeros.
    """
    B, Hq, Tq, D = query.shape
    o, lse = _AttnMasked.apply(_rows(query), _rows(key), _rows(value), mask, B, float(scale))
    o = o.view(B, Tq, Hq, D)
    return (o, lse) if return_lse else o


class DuoMask:
    """What the dense mask of tah_model.py:744-791 is computed from, kept symbolic."""

    def __init__(self, position_ids: torch.Tensor, valid_mask: torch.Tensor, cache: Optional[TaHDuoCache], iter_depth: int):
        self.position_ids, self.valid_mask, self.cache, self.iter_depth = position_ids, valid_mask, cache, iter_depth
        self._packed = None  # per-step packing metadata, shared by all decoder layers
        self._sched = None   # launch-order table of the step's varlen calls, likewise
        self._merge = None   # where the rows of depths 1 .. iter_depth go in their common packing (depth >= 2)

    def dense(self, dtype: torch.dtype = torch.float32) -> Optional[torch.Tensor]:
        """The (B,1,Tq,Tkv) additive mask the reference would have built (for inspection only)."""
        B, T = self.position_ids.shape
        c, d, dev = self.cache, self.iter_depth, self.position_ids.device
        if c is not None and c.has_layer(0):
            it = c.get_cache_iter_index_upto_iter(0, d)
            pos = c.get_position_id_upto_iter(0, d, B)
            val = c.get_valid_mask_upto_iter(0, d, B)
        else:
            it = torch.empty((0,), dtype=torch.long, device=dev)
            pos = torch.empty((B, 0), dtype=torch.long, device=dev)
            val = torch.empty((B, 0), dtype=torch.long, device=dev)
        if it.numel() + T == 0:
            return None
        kv_pos = torch.cat((pos, self.position_ids), -1)[:, None, :]
        kv_val = torch.cat((val, self.valid_mask), -1)[:, None, :]
        kv_it = torch.cat((it, torch.full((T,), d, dtype=torch.long, device=dev)))[None, None, :]
        see = (kv_pos <= self.position_ids[:, :, None]) & (kv_it <= d) & (kv_val == 1)
        m = torch.full(see.shape, torch.finfo(dtype).min, dtype=dtype, device=dev)
        m[see] = 0.0
        return m[:, None]


def build_attention_mask(active_position_ids, active_valid_mask, cache, iter_depth, dtype=None) -> Optional[DuoMask]:
    """Drop-in for ``TaHForCausalLM._build_attention_mask`` (tah_model.py:744-751): same arguments;
    returns a :class:`DuoMask` (or ``None`` when there is nothing to attend to, as tah_model.py:773-775)."""
    del dtype
    _check_depth(iter_depth)
    n_cached = cache.get_kv_length_upto_iter(0, iter_depth) if cache is not None and cache.has_layer(0) else 0
    if n_cached + active_position_ids.shape[1] == 0:
        return None
    return DuoMask(active_position_ids, active_valid_mask, cache, iter_depth)


def _check_depth(iter_depth: int) -> None:
    """Any latent depth is accepted, as the reference's mask accepts it (tah_model.py:788): a query at depth d sees the
    keys at or before its position of every depth <= d."""
    if int(iter_depth) < 0:
        raise TahDuoError(f"iter_depth = {iter_depth}: a latent iteration depth cannot be negative")


# Debug switch: verify on the device (one host sync per model step) that the positions handed in are the
# valid tokens' ranks inside their sequence -- what the kernels assume for depth 0 (index-causal order) and
# for the depth-0 keys that depth-1 queries see.  The model's forward computes exactly these when
# ``position_ids`` is None (tah_model.py:555-561); a caller that passes its own position_ids can turn this on.
CHECK_POSITIONS = False

# What the positions handed to ``build_attention_mask`` are.  True: the rank of a valid token inside its sequence, which
# the model's forward computes when ``position_ids`` is None (tah_model.py:555-561); depth-0 keys then need no
# position (it is their index) and the kernels skip the key tiles behind a query tile.  False: plain numbers that the
# caller chose (tah_model.py:499 hands ``position_ids`` through and :788 compares them as they are): every key then
# carries its position -- depth-0 rows go through the position-carrying stream as well, any order and any repeats,
# at the price of visiting every (query tile, key tile) pair of a sequence.  Packed path only: the decode path's
# depth-0 slabs keep no positions.
POSITION_IDS_ARE_RANKS = True


def _assert_rank_positions(m: "DuoMask") -> None:
    c, B = m.cache, m.position_ids.shape[0]
    prev = 0
    if c is not None and c.has_layer(0):
        # valid depth-0 tokens already cached (the step's own rows are written by update() before attention runs)
        cached = c.get_valid_mask_upto_iter(0, 0, B)
        own = m.valid_mask.shape[1] if m.iter_depth == 0 and cached.shape[1] >= m.valid_mask.shape[1] else 0
        prev = cached[:, : cached.shape[1] - own].sum(-1, keepdim=True) if cached.shape[1] - own > 0 else 0
    v = m.valid_mask != 0
    if m.iter_depth == 0:
        want = torch.cumsum(v.long(), -1) - 1 + prev
        bad = ((m.position_ids != want) & v).any()
    else:  # depth-1 rows name tokens that exist at depth 0: positions below the number of valid depth-0 tokens
        total0 = c.get_valid_mask_upto_iter(0, 0, B).sum(-1, keepdim=True)
        bad = (((m.position_ids < 0) | (m.position_ids >= total0)) & v).any()
    if bool(bad):
        raise TahDuoError("position_ids are not the valid tokens' ranks inside their sequence; the kernels take the "
                          "depth-0 position of a token from its index among the valid tokens "
                          "(tah_amd.attention.POSITION_IDS_ARE_RANKS = False makes every key carry its position instead)")


# ---------------------------------------------------------------------------
# packing helpers
# ---------------------------------------------------------------------------


def _rows(x: torch.Tensor) -> torch.Tensor:
    """(B, H, T, D) -> [B*T, H, D]; free when x is the usual transposed view of a (B,T,H,D) projection."""
    B, H, T, D = x.shape
    return x.transpose(1, 2).reshape(B * T, H, D)


# Blocks of at most this many rows are packed without reading their valid count back (see _Packed).
NO_SYNC_ROWS = 4096


class _Packed:
    """Valid-row packing of one (B, T) block: row ids, per-sequence offsets, int32 positions.

    With ``tah_amd.pack.HOST_SYNC`` off nothing is read back from the device: packed tensors keep the full
    B*T rows (zero beyond the valid count, so that a key tile never mixes in uninitialised rows), the kernels
    find the real extent in ``cu``, and the row copies stop at the count held on the device."""

    def __init__(self, valid: Optional[torch.Tensor], pos: Optional[torch.Tensor], B: int, T: int, device):
        self.B, self.T = B, T
        self.n_dev = None
        if valid is not None and tuple(valid.shape) != (B, T):
            raise TahDuoError(f"valid mask of shape {tuple(valid.shape)} for a block of {B} x {T} rows")
        if pos is not None and pos.numel() != B * T:
            raise TahDuoError(f"positions of shape {tuple(pos.shape)} for a block of {B} x {T} rows")
        all_valid = valid is None
        if not all_valid:
            # a small block (the packed hard tokens of a step) is packed by its upper bound, B * T rows: reading the count
            # back would stall the host on everything queued so far to save copying a few pad rows
            idx = HardIndex.of(valid, sync=None if B * T > NO_SYNC_ROWS else False)
            all_valid = idx.synced and idx.n == B * T
        if all_valid:
            self.rows, self.n = None, B * T
            self.cu = torch.arange(0, (B + 1) * T, T, dtype=torch.int32, device=device)
        else:
            self.rows, self.n, self.cu, self.n_dev = idx.flat, idx.bound, idx.cu, idx.n_dev
        self.pos = None
        if pos is not None:
            p32 = pos.to(torch.int32).contiguous().view(B * T, 1)
            if self.rows is not None:
                out = torch.zeros((self.n, 1), dtype=torch.int32, device=device)
                ops.rows_copy(p32, self.rows, out, None, self.n, None, self.n_dev)
                p32 = out
            self.pos = p32.view(-1)

    def pack(self, x: torch.Tensor) -> torch.Tensor:
        r = _rows(x)
        if self.rows is None:
            return r
        return _GatherRows.apply(r.contiguous(), self.rows, self.n, self.n_dev)

    def unpack(self, o: torch.Tensor, Hq: int, D: int) -> torch.Tensor:
        """[n, Hq, D] -> (B, T, Hq, D) with zeros at rows that were not packed."""
        if self.rows is None:
            return o.view(self.B, self.T, Hq, D)
        return _ScatterRows.apply(o, self.rows, self.n, self.B * self.T, self.n_dev).view(self.B, self.T, Hq, D)


class _GatherRows(torch.autograd.Function):
    @staticmethod
    def forward(ctx, src, rows, n, n_dev=None):
        alloc = torch.empty if n_dev is None else torch.zeros  # rows past a device-side count stay zero
        out = alloc((n,) + tuple(src.shape[1:]), dtype=src.dtype, device=src.device)
        ops.rows_copy(src, rows, out, None, n, None, n_dev)
        ctx.save_for_backward(rows, n_dev)
        ctx.n, ctx.total = n, src.shape[0]
        return out

    @staticmethod
    def backward(ctx, g):
        rows, n_dev = ctx.saved_tensors
        gs = torch.zeros((ctx.total,) + tuple(g.shape[1:]), dtype=g.dtype, device=g.device)
        ops.rows_copy(g.contiguous(), None, gs, rows, ctx.n, None, n_dev)
        return gs, None, None, None


class _ScatterRows(torch.autograd.Function):
    @staticmethod
    def forward(ctx, src, rows, n, total, n_dev=None):
        out = torch.zeros((total,) + tuple(src.shape[1:]), dtype=src.dtype, device=src.device)
        ops.rows_copy(src.contiguous(), None, out, rows, n, None, n_dev)
        ctx.save_for_backward(rows, n_dev)
        ctx.n = n
        return out

    @staticmethod
    def backward(ctx, g):
        rows, n_dev = ctx.saved_tensors
        alloc = torch.empty if n_dev is None else torch.zeros
        gs = alloc((ctx.n,) + tuple(g.shape[1:]), dtype=g.dtype, device=g.device)
        ops.rows_copy(g.contiguous(), rows, gs, None, ctx.n, None, n_dev)
        return gs, None, None, None, None


def _segment(cache: TaHDuoCache, layer_idx: int, depth: int, B: int, with_pos: bool):
    """All rows written at (layer, depth), packed per sequence: k, v [rows,Hkv,D], cu int32, pos int32 or None.

    One chunk (prefill / training, the only case on the backward path) packs without copies when every
    token is valid; several chunks (a cache grown by earlier calls) are concatenated per sequence.
    """
    chunks = cache.chunks(layer_idx, depth)
    if not chunks:
        raise TahDuoError(f"no keys cached for layer {layer_idx} at depth {depth}")
    dev = chunks[0][0].device
    if len(chunks) == 1:
        k, v, pos, valid = chunks[0]
        # every decoder layer caches the same (valid, pos) tensors of the step: build the index once
        key = (id(valid), id(pos) if with_pos else None, k.shape[2])
        memo = cache._key_memo.get(key)
        if memo is None or memo[0] is not valid or (with_pos and memo[1] is not pos):
            memo = (valid, pos, _Packed(valid, pos if with_pos else None, B, k.shape[2], dev))
            if len(cache._key_memo) > 8:
                cache._key_memo.clear()
            cache._key_memo[key] = memo
        pk = memo[2]
        # The packed rows themselves are kept per (layer, depth): the calls of later depths attend over the same chunk,
        # and under autograd their gradients then meet at the packed tensor (one scatter back, not one per call).
        # (Training only: without gradients the copy would only hold memory for as long as the cache lives.)
        if pk.rows is None or not (torch.is_grad_enabled() and (k.requires_grad or v.requires_grad)):
            return pk.pack(k), pk.pack(v), pk.cu, pk.pos
        slot = (layer_idx, depth)
        kept = cache._kv_packed.get(slot)
        if kept is None or kept[0] is not k or kept[1] is not v or kept[2] is not pk or kept[3] != (k._version, v._version):
            kept = (k, v, pk, (k._version, v._version), pk.pack(k), pk.pack(v))
            cache._kv_packed[slot] = kept
        return kept[4], kept[5], pk.cu, pk.pos
    k = torch.cat([c[0] for c in chunks], dim=2)
    v = torch.cat([c[1] for c in chunks], dim=2)
    T = k.shape[2]
    one = lambda c, fill: (torch.full((B, c[0].shape[2]), fill, dtype=torch.long, device=dev))
    valid = torch.cat([c[3] if c[3] is not None else one(c, 1) for c in chunks], dim=1)
    pos = torch.cat([c[2] if c[2] is not None else one(c, 0) for c in chunks], dim=1) if with_pos else None
    pk = _Packed(valid, pos, B, T, dev)
    return pk.pack(k), pk.pack(v), pk.cu, pk.pos


def _merge_plan(m: "DuoMask", segs, B: int):
    """Where the rows of several packed segments go when they are packed together, sequence by sequence (inside a
    sequence: the first segment's rows, then the second's, ...): (dest int64 [sum of rows], cu int32 [B+1], pos int32).
    Built on the device from the segments' boundaries, once per step (every layer caches the same boundaries).  Rows
    past a segment's cu[B] (packing by upper bounds) go past the merged cu[B]."""
    key = tuple((sg[2].data_ptr(), sg[0].shape[0]) for sg in segs)
    memo = getattr(m, "_merge", None)
    if memo is not None and memo[0] == key:
        return memo[1:]
    dev = segs[0][2].device
    cus = [sg[2].long() for sg in segs]
    cu_m = torch.stack(cus).sum(0)
    off = torch.zeros(B, dtype=torch.long, device=dev)
    tail = cu_m[B]
    dests = []
    for cu, sg in zip(cus, segs):
        n = sg[0].shape[0]
        r = torch.arange(n, dtype=torch.long, device=dev)
        seq = torch.searchsorted(cu[1:].contiguous(), r, right=True)
        sq = seq.clamp(max=B - 1)
        dests.append(torch.where(seq < B, cu_m[sq] + off[sq] + (r - cu[sq]), tail + (r - cu[B])))
        off = off + (cu[1:] - cu[:-1])
        tail = tail + (n - cu[B])
    dest = torch.cat(dests)
    pos = torch.zeros(dest.shape[0], dtype=torch.int32, device=dev).index_copy_(0, dest, torch.cat([sg[3] for sg in segs]))
    m._merge = (key, dest, cu_m.to(torch.int32), pos)
    return m._merge[1:]


def _sparse_keys(m: "DuoMask", cache: TaHDuoCache, layer: int, depth: int, B: int, first: int = 1):
    """The keys a query at ``depth`` >= 1 sees beside the depth-0 ones: every row cached at depths 1 .. depth (``first``
    = 0: with the depth-0 rows, for positions that are not ranks), packed per
    sequence with their positions -- (k, v, cu, pos, upper bound of a sequence's rows).  The kernels tell depth-0 keys
    (position = index) from keys that carry a position, and among the latter a query sees those at or before its own
    position whatever their depth (tah_model.py:788 with depth_k <= depth_q for all of them), so deeper calls hand the
    kernels the union of these depths as the one sparse key stream; one depth needs no copy."""
    segs = [_segment(cache, layer, d, B, with_pos=True) for d in range(first, depth + 1) if cache.has_rows(layer, d)]
    if not segs:
        raise TahDuoError(f"no keys cached for layer {layer} at depths {first}..{depth}")
    bound = sum(cache.get_cache_length(layer, d) for d in range(first, depth + 1))
    if len(segs) == 1:
        return segs[0] + (bound,)
    dest, cu, pos = _merge_plan(m, segs, B)
    kcat, vcat = torch.cat([sg[0] for sg in segs]), torch.cat([sg[1] for sg in segs])
    return torch.zeros_like(kcat).index_copy(0, dest, kcat), torch.zeros_like(vcat).index_copy(0, dest, vcat), cu, pos, bound


def duo_attention_forward(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                          attention_mask, dropout: float = 0.0, scaling: Optional[float] = None,
                          is_causal: Optional[bool] = None, **kwargs) -> Tuple[torch.Tensor, None]:
    """Hugging Face attention-interface callable for duo-causal attention.

    query (B,Hq,Tq,D); key/value are whatever ``cache.update`` returned (the new rows); ``attention_mask``
    is the :class:`DuoMask` built for this step; ``module.layer_idx`` names the layer.  Returns
    ``(attn_output (B,Tq,Hq,D), None)`` like sdpa_attention_forward (sdpa_attention.py:164-166).
    A dense additive tensor in the mask slot (what tah_model.py:744-791 builds) selects the compatibility
    mode instead: key/value must then be the full (B,Hkv,Tkv,D) tensors the mask's last axis runs over,
    as the reference's ``cache.update`` returns them, and the result is that of SDPA with this mask.
    """
    del is_causal, kwargs
    if torch.is_tensor(attention_mask):
        if dropout:
            raise TahDuoError("attention dropout is not supported (the reference runs with 0.0)")
        if attention_mask.dim() != 4 or key.shape[2] != attention_mask.shape[-1]:
            raise TahDuoError("a dense attention mask must be 4-D with its last axis over the rows of key/value "
                              f"(mask {tuple(attention_mask.shape)}, key {tuple(key.shape)})")
        D = query.shape[-1]
        m = attention_mask
        if m.dtype not in (torch.bfloat16, torch.float32):
            m = m.to(torch.float32)
        return attn_additive_mask(query, key, value, m, float(scaling) if scaling is not None else float(D) ** -0.5), None
    if not isinstance(attention_mask, DuoMask):
        raise TahDuoError("duo_attention_forward needs the DuoMask from tah_amd.attention.build_attention_mask (or the "
                          "reference's dense additive mask) in the attention_mask slot")
    if dropout:
        raise TahDuoError("attention dropout is not supported (the reference runs with 0.0)")
    m = attention_mask
    cache, depth = m.cache, m.iter_depth
    _check_depth(depth)
    if CHECK_POSITIONS and POSITION_IDS_ARE_RANKS and m._packed is None:
        _assert_rank_positions(m)
    if cache is None:
        raise TahDuoError("the DuoMask carries no cache; pass the cache that update() was called on")
    layer = int(getattr(module, "layer_idx", 0))
    B, Hq, Tq, D = query.shape
    scale = float(scaling) if scaling is not None else float(D) ** -0.5
    dev = query.device

    # decode fast path: one query row per sequence, slabs hold every cached row (incl. this step's)
    s1 = cache.slabs(layer, 0)
    ranks = POSITION_IDS_ARE_RANKS
    if s1 is not None and not ranks:
        raise TahDuoError("POSITION_IDS_ARE_RANKS = False: position ids of the caller's choosing run on the packed path only "
                          "(the decode path's depth-0 slabs keep no positions); use a cache without enable_slabs()")
    if Tq == 1 and s1 is not None and depth <= 1 and not (torch.is_grad_enabled() and query.requires_grad):
        # every batch row is a query row; a row that is not valid (a pad row of the depth-1 pack, tah_model.py:116-118)
        # gets position -1, sees nothing and comes back as zeros -- no index to build, nothing read back
        if m._packed is None:
            pos32 = m.position_ids.to(torch.int32).reshape(B)
            qpos = torch.where(m.valid_mask.reshape(B) != 0, pos32, torch.full_like(pos32, -1))
            m._packed = (torch.arange(B, dtype=torch.int32, device=dev), qpos)
        slots, qpos = m._packed
        o = kv_cache.decode(_rows(query), slots, qpos, s1, cache.slabs(layer, 1) if depth >= 1 else None, scale=scale,
                            depth=depth)
        return o.view(B, 1, Hq, D), None

    # general path: packed varlen forward (+ backward through autograd)
    if m._packed is None:
        m._packed = _Packed(m.valid_mask, m.position_ids if (depth >= 1 or not ranks) else None, B, Tq, dev)
    pq = m._packed
    if not isinstance(pq, _Packed):
        raise TahDuoError("a DuoMask cannot be shared between the decode path and the varlen path")
    q = pq.pack(query)
    zc = torch.zeros(B + 1, dtype=torch.int32, device=dev)
    zi = torch.zeros(0, dtype=torch.int32, device=dev)
    e_q = q[:0]
    if depth == 0 and ranks:
        k1, v1, cu_k1, _ = _segment(cache, layer, 0, B, with_pos=False)
        Hkv = k1.shape[1]
        e_k = k1[:0]
        sched = _schedule_of(m, (pq.cu, cu_k1, zc, zc, zi, Hq, Hkv, q.shape[0], k1.shape[0], 0))
        o, _ = duo_attn_varlen(q, k1, v1, pq.cu, cu_k1, e_q, e_k, e_k, zi, zi, zc, zc, scale, schedule=sched,
                               max_seqlen_k1=cache.get_cache_length(layer, 0))
    else:
        k2, v2, cu_k2, pos_k2, bound_k2 = _sparse_keys(m, cache, layer, depth, B, first=1 if ranks else 0)
        Hkv = k2.shape[1]
        if ranks:
            k1, v1, cu_k1, _ = _segment(cache, layer, 0, B, with_pos=False)
            bound_k1 = cache.get_cache_length(layer, 0)
        else:  # no key without a position of its own
            k1, v1, cu_k1, bound_k1 = k2[:0], v2[:0], zc, 0
        sched = _schedule_of(m, (zc, cu_k1, pq.cu, cu_k2, pq.pos, Hq, Hkv, 0, k1.shape[0], k2.shape[0]))
        _, o = duo_attn_varlen(e_q, k1, v1, zc, cu_k1, q, k2, v2, pq.pos, pos_k2, pq.cu, cu_k2, scale, schedule=sched,
                               max_seqlen_k1=bound_k1, max_seqlen_k2=bound_k2)
    return pq.unpack(o, Hq, D), None


# Calls with at least this many (query row, kv head) pairs get a launch-order table: below it a launch has about
# one workgroup per compute unit and the order does not matter.  Nor does it for a batch of short sequences (every tile
# runs a step or two; measured: 64 x 128 tokens lose 25 % of the forward to the table, 16 x 512 gain 12 % of the
# backward): the table is for batches whose sequences average at least SCHEDULE_MIN_MEAN_ROWS query rows.
SCHEDULE_MIN_ROW_HEADS = 49152
SCHEDULE_MIN_MEAN_ROWS = 256


def _schedule_of(m: "DuoMask", args):
    """The launch-order table of this mask's varlen calls: built at the first layer, shared by the others (the
    boundaries of queries and cached keys are the same in every layer of a step) and by the backward pass."""
    cu_q1, cu_k1, cu_q2, cu_k2, pos_q2, hq, hkv, tq1, tk1, tk2 = args
    rows, nseq = tq1 + pos_q2.shape[0], max(1, cu_k1.numel() - 1)
    if rows * hkv < SCHEDULE_MIN_ROW_HEADS or rows < SCHEDULE_MIN_MEAN_ROWS * nseq:
        return None
    key = (tq1, tk1, pos_q2.shape[0], tk2, hq, hkv, cu_k1.data_ptr(), cu_k2.data_ptr())
    memo = getattr(m, "_sched", None)
    if memo is None or memo[0] != key:
        memo = (key, ops.duo_schedule(cu_q1, cu_k1, cu_q2, cu_k2, pos_q2, hq, hkv, tq1, tk1, tk2), (cu_k1, cu_k2))
        m._sched = memo
    return memo[1]


def register_with_transformers(name: str = "tah_duo") -> str:
    """Register :func:`duo_attention_forward` under ``attn_implementation=name`` (needs transformers)."""
    from transformers import AttentionInterface

    AttentionInterface.register(name, duo_attention_forward)
    return name
