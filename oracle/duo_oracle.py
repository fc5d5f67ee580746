"""CPU oracle for TaH duo-causal attention.  TEST INFRASTRUCTURE ONLY.

Nothing under ``tah_amd/`` may import this module: it exists so that tests,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` have an
independent statement of what the HIP kernels must compute.

Two statements of the algorithm live here and are checked against each other
and against closed forms by ``tests/test_oracle.py``:

* the *dense* restatement, which follows the reference's formulation step by
  step (additive mask -> GQA expansion -> softmax(QK^T s + M) V, with a
  list-append KV cache), and
* the *row-loop* restatement (:func:`duo_rows_f64`), float64, which evaluates
  the visibility predicate pair by pair on the packed varlen layout that the
  HIP kernels consume, and shares no code with the dense one.

Parity status per function (what pins it):

=====================  ==========================================================
function               pinned by
=====================  ==========================================================
duo_visible            triple-loop brute force; reduces to plain causal when no
                       key is at depth 1
build_attention_mask   brute force over (b, i, j); p=0 => torch causal mask
OracleCache            property: update() == cat of writes with depth <= current
repeat_kv              equals torch.repeat_interleave
sdpa_dense             torch.nn.functional.scaled_dot_product_attention (library
                       routine) incl. is_causal=True special case; float64 rows
gather_active /        mask.nonzero() order; round-trip identities
scatter_back
duo_prefill_dense      agreement with duo_rows_f64 (independent code)
gradients              torch autograd on the dense path vs the analytic C
                       backward in duo_ref.c vs central finite differences
=====================  ==========================================================

The reference ships no golden vectors or tests for this path and its arithmetic
lives in un-vendored third-party code (transformers==4.52.4, torch==2.6.0,
pyproject.toml:21-22), so the fixtures under tests/golden/ are produced from
these two restatements after they agree.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

# --------------------------------------------------------------------------
# Visibility predicate and mask   (tah/model/tah_model.py:744-791)
# --------------------------------------------------------------------------


def duo_visible(q_pos: int, q_iter: int, kv_pos: int, kv_iter: int, kv_valid: int = 1) -> bool:
    """Key (kv_pos, kv_iter) is visible to query (q_pos, q_iter).

    tah/model/tah_model.py:788 -- ``(kv_pos <= q_pos) & (kv_iter <= q_iter) & (kv_valid == 1)``.
    """
    return bool(kv_pos <= q_pos and kv_iter <= q_iter and kv_valid == 1)


class OracleCache:
    """List-append model of ``TaHCache`` (tah/model/causal_cache.py:30-239).

    One list of writes per (layer, depth).  ``update`` appends and returns the
    depth-major concatenation of everything at depth <= current
    (causal_cache.py:63-109).
    """

    def __init__(self) -> None:
        self.k: Dict[Tuple[int, int], List[torch.Tensor]] = {}
        self.v: Dict[Tuple[int, int], List[torch.Tensor]] = {}
        self.pos: Dict[Tuple[int, int], List[torch.Tensor]] = {}
        self.valid: Dict[Tuple[int, int], List[torch.Tensor]] = {}
        self.current_iter_depth = 0
        self.position_ids_to_cache: Optional[torch.Tensor] = None
        self.valid_mask_to_cache: Optional[torch.Tensor] = None
        self.batch_size: Optional[int] = None

    def has_layer(self, layer_idx: int = 0) -> bool:  # causal_cache.py:57-59
        return any(l == layer_idx for (l, _) in self.k)

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        if self.batch_size is None:
            self.batch_size = key_states.shape[0]
        elif key_states.shape[0] != self.batch_size:  # causal_cache.py:79-81
            raise AssertionError("batch size mismatch")
        slot = (layer_idx, self.current_iter_depth)
        self.k.setdefault(slot, []).append(key_states)
        self.v.setdefault(slot, []).append(value_states)
        self.pos.setdefault(slot, []).append(self.position_ids_to_cache)
        self.valid.setdefault(slot, []).append(self.valid_mask_to_cache)
        return self.get_cache_upto_iter(layer_idx, self.current_iter_depth)

    def get_cache_upto_iter(self, layer_idx, upto_iter_idx):  # causal_cache.py:101-109
        ks, vs = [], []
        for d in range(upto_iter_idx + 1):
            ks += self.k.get((layer_idx, d), [])
            vs += self.v.get((layer_idx, d), [])
        if not ks:
            return None, None
        return torch.cat(ks, dim=-2), torch.cat(vs, dim=-2)

    def _meta(self, store, layer_idx, upto, batch):  # causal_cache.py:111-134
        parts = []
        for d in range(upto + 1):
            parts += store.get((layer_idx, d), [])
        if not parts:
            return torch.empty((batch, 0), dtype=torch.long)
        return torch.cat(parts, dim=-1)

    def get_position_id_upto_iter(self, layer_idx, upto_iter_idx, init_batch_size=1):
        return self._meta(self.pos, layer_idx, upto_iter_idx, init_batch_size)

    def get_valid_mask_upto_iter(self, layer_idx, upto_iter_idx, init_batch_size=1):
        return self._meta(self.valid, layer_idx, upto_iter_idx, init_batch_size)

    def get_cache_iter_index_upto_iter(self, layer_idx, upto_iter_idx):  # causal_cache.py:142-158
        out = []
        for d in range(upto_iter_idx + 1):
            n = sum(t.shape[-2] for t in self.k.get((layer_idx, d), []))
            out += [d] * n
        return torch.tensor(out, dtype=torch.long)

    def get_cache_length(self, layer_idx=0, iter_idx=None):  # causal_cache.py:162-167
        tot = 0
        for (l, d), ts in self.k.items():
            if l == layer_idx and (iter_idx is None or d == iter_idx):
                tot += sum(t.shape[-2] for t in ts)
        return tot

    def get_kv_length_upto_iter(self, layer_idx=0, upto_iter_idx=0):  # causal_cache.py:169-181
        return sum(self.get_cache_length(layer_idx, d) for d in range(upto_iter_idx + 1))

    def get_seq_length(self, layer_idx=0, iter_idx=0):  # causal_cache.py:183-186
        return self.get_cache_length(layer_idx, iter_idx)


def build_attention_mask(
    active_position_ids: torch.Tensor,
    active_valid_mask: torch.Tensor,
    cache: Optional[OracleCache],
    iter_depth: int,
    dtype: torch.dtype,
) -> Optional[torch.Tensor]:
    """Additive mask ``(B, 1, Tq, Tkv)`` (tah/model/tah_model.py:744-791).

    kv axis = cached slots at depth 0..iter_depth (depth-major), then the Tq
    rows being written at ``iter_depth`` (:778-783).  Visible -> 0, else
    ``finfo(dtype).min`` (:776, :789-790).  ``None`` when the kv axis is empty
    (:773-775).
    """
    B, T = active_position_ids.shape
    if cache is not None and cache.has_layer(0):
        c_iter = cache.get_cache_iter_index_upto_iter(0, iter_depth)
        c_pos = cache.get_position_id_upto_iter(0, iter_depth, B)
        c_valid = cache.get_valid_mask_upto_iter(0, iter_depth, B)
    else:
        c_iter = torch.empty((0,), dtype=torch.long)
        c_pos = torch.empty((B, 0), dtype=torch.long)
        c_valid = torch.empty((B, 0), dtype=torch.long)
    n_kv = c_iter.numel() + T
    if n_kv == 0:
        return None
    kv_pos = torch.cat([c_pos, active_position_ids], dim=1)
    kv_valid = torch.cat([c_valid, active_valid_mask], dim=1)
    kv_iter = torch.cat([c_iter, torch.full((T,), iter_depth, dtype=torch.long)])
    see = (
        (kv_pos[:, None, :] <= active_position_ids[:, :, None])
        & (kv_iter[None, None, :] <= iter_depth)
        & (kv_valid[:, None, :] == 1)
    )
    neg = torch.finfo(dtype).min
    m = torch.where(see, torch.zeros((), dtype=dtype), torch.full((), neg, dtype=dtype))
    return m[:, None]


# --------------------------------------------------------------------------
# Attention arithmetic (third-party in the reference:
# transformers/integrations/sdpa_attention.py:15-24, 79-166 + torch SDPA)
# --------------------------------------------------------------------------


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """(B, Hkv, T, D) -> (B, Hkv*n_rep, T, D); q head h reads kv head h // n_rep."""
    if n_rep == 1:
        return x
    b, h, t, d = x.shape
    return x.unsqueeze(2).expand(b, h, n_rep, t, d).reshape(b, h * n_rep, t, d)


def sdpa_dense(q, k, v, mask, scale) -> torch.Tensor:
    """softmax(q k^T * scale + mask) v, GQA by expansion; returns (B, Tq, Hq, D).

    q (B,Hq,Tq,D); k,v (B,Hkv,Tkv,D); mask broadcastable to (B,Hq,Tq,Tkv) or None.
    Softmax is taken in the dtype of q (use float32/float64 inputs).
    """
    g = q.shape[1] // k.shape[1]
    kk, vv = repeat_kv(k, g), repeat_kv(v, g)
    s = torch.matmul(q, kk.transpose(-1, -2)) * scale
    if mask is not None:
        s = s + mask
    p = torch.softmax(s, dim=-1)
    return torch.matmul(p, vv).transpose(1, 2).contiguous()


# --------------------------------------------------------------------------
# Hard-token pack / scatter   (tah/model/tah_model.py:96-176)
# --------------------------------------------------------------------------


def hard_index(mask: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Packed-varlen form of a (B, S) bool mask.

    idx[r]  = position (column) of the r-th True in row-major order, int32;
    cu[b]   = number of True entries in rows < b, int32, length B+1.
    Row-major order is the order of tah_model.py:114-117 / :163-167.
    """
    nz = mask.nonzero()
    idx = nz[:, 1].to(torch.int32)
    cu = torch.zeros(mask.shape[0] + 1, dtype=torch.int32)
    cu[1:] = torch.cumsum(mask.sum(1), 0).to(torch.int32)
    return idx, cu


def gather_active(current_iter_mask: torch.Tensor, *tensors, pad_value=0):
    """Left-pack the True positions of each row (tah_model.py:96-135).

    Returns ``(pad_mask, *gathered)``; gathered tensors are (B, max_active, ...)
    with pads filled with ``pad_value``; ``None`` inputs pass through.
    Restated with explicit per-row index lists instead of the stable sort.
    """
    B, S = current_iter_mask.shape
    rows = [torch.nonzero(current_iter_mask[b]).flatten() for b in range(B)]
    width = max((len(r) for r in rows), default=0)
    pad_mask = torch.ones((B, width), dtype=torch.bool)
    for b, r in enumerate(rows):
        pad_mask[b, : len(r)] = False
    out = [pad_mask]
    for t in tensors:
        if t is None:
            out.append(None)
            continue
        g = torch.full((B, width) + tuple(t.shape[2:]), pad_value, dtype=t.dtype)
        for b, r in enumerate(rows):
            if len(r):
                g[b, : len(r)] = t[b, r]
        out.append(g)
    return tuple(out)


def scatter_back(current_iter_mask, src, dest, *, in_place=False, assignment_mask=None):
    """Inverse of :func:`gather_active` (tah_model.py:138-176)."""
    out = dest if in_place else dest.clone()
    B = current_iter_mask.shape[0]
    for b in range(B):
        cols = torch.nonzero(current_iter_mask[b]).flatten()
        for k, c in enumerate(cols.tolist()):
            if assignment_mask is None or bool(assignment_mask[b, c]):
                out[b, c] = src[b, k]
    return out


# --------------------------------------------------------------------------
# The whole op, dense formulation, as the reference's forward loop drives it
# (tah_model.py:580-623 for depth 0 then depth 1)
# --------------------------------------------------------------------------


def duo_prefill_dense(q1, k1, v1, q2_dense, k2_dense, v2_dense, hard_mask, scale,
                      valid_mask=None, position_ids=None):
    """Two-depth duo-causal attention over a (B, T) batch, dense formulation.

    q1 (B,Hq,T,D), k1/v1 (B,Hkv,T,D): depth-0 projections of every token.
    q2_dense/k2_dense/v2_dense: depth-1 projections laid out densely (B,H,T,D);
    only rows where ``hard_mask`` (B,T) is True are used.
    Returns ``o1 (B,T,Hq,D)``, ``o2 (B,max_active,Hq,D)``, ``pad_mask``.
    """
    B, _, T, _ = q1.shape
    if valid_mask is None:
        valid_mask = torch.ones((B, T), dtype=torch.long)
    if position_ids is None:  # tah_model.py:555-559 with an empty cache
        position_ids = (torch.cumsum(valid_mask, -1) - 1).clamp(min=0)
    cache = OracleCache()
    # depth 0: every token is active
    m0 = build_attention_mask(position_ids, valid_mask, cache, 0, q1.dtype)
    cache.current_iter_depth = 0
    cache.position_ids_to_cache = position_ids
    cache.valid_mask_to_cache = valid_mask
    K, V = cache.update(k1, v1, 0)
    o1 = sdpa_dense(q1, K, V, m0, scale)
    # depth 1: hard tokens only, left-packed per row
    tok = lambda x: x.transpose(1, 2)  # (B,H,T,D) -> (B,T,H,D) so gather runs over dim 1
    pad, q2, k2, v2, pos2, val2 = gather_active(
        hard_mask, tok(q2_dense), tok(k2_dense), tok(v2_dense), position_ids, valid_mask)
    if pad.shape[1] == 0:
        return o1, q1.new_zeros((B, 0, q1.shape[1], q1.shape[3])), pad
    m1 = build_attention_mask(pos2, val2, cache, 1, q1.dtype)
    cache.current_iter_depth = 1
    cache.position_ids_to_cache = pos2
    cache.valid_mask_to_cache = val2
    K, V = cache.update(tok(k2), tok(v2), 0)
    o2 = sdpa_dense(tok(q2), K, V, m1, scale)
    return o1, o2, pad


# --------------------------------------------------------------------------
# Independent float64 statement on the packed varlen layout
# --------------------------------------------------------------------------


def duo_rows_f64(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale):
    """Row-by-row duo-causal attention on packed varlen inputs, float64 numpy.

    q1 (T1q,Hq,D), k1/v1 (T1k,Hkv,D); q2 (T2q,Hq,D), k2/v2 (T2k,Hkv,D).
    In sequence b, depth-0 key j (local index) has position j; depth-0 query i
    has position ``i + (Lk1_b - Lq1_b)``; depth-1 rows carry explicit positions.
    Visibility is :func:`duo_visible`, evaluated pair by pair.
    Returns o1, lse1 (Hq,T1q), o2, lse2 (Hq,T2q); lse is the natural-log
    normaliser of the scaled scores.
    """
    f = lambda x: np.asarray(x, dtype=np.float64)
    q1, k1, v1, q2, k2, v2 = map(f, (q1, k1, v1, q2, k2, v2))
    cu_q1, cu_k1, cu_q2, cu_k2 = (np.asarray(c, dtype=np.int64) for c in (cu_q1, cu_k1, cu_q2, cu_k2))
    pos_q2 = np.asarray(pos_q2, dtype=np.int64)
    pos_k2 = np.asarray(pos_k2, dtype=np.int64)
    Hq, D = q1.shape[1], q1.shape[2]
    g = Hq // k1.shape[1]
    o1 = np.zeros_like(q1)
    o2 = np.zeros_like(q2)
    lse1 = np.full((Hq, q1.shape[0]), -np.inf)
    lse2 = np.full((Hq, q2.shape[0]), -np.inf)
    nseq = len(cu_q1) - 1

    def one_row(qrow, keys, vals):
        s = keys @ qrow * scale
        m = s.max()
        e = np.exp(s - m)
        return (e @ vals) / e.sum(), m + np.log(e.sum())

    for b in range(nseq):
        a0, a1 = cu_q1[b], cu_q1[b + 1]
        c0, c1 = cu_k1[b], cu_k1[b + 1]
        off = (c1 - c0) - (a1 - a0)
        e0, e1 = cu_k2[b], cu_k2[b + 1]
        for h in range(Hq):
            hk = h // g
            for i in range(a0, a1):
                p = (i - a0) + off
                sel = [j for j in range(c0, c1) if duo_visible(p, 0, j - c0, 0)]
                if sel:
                    o1[i, h], lse1[h, i] = one_row(q1[i, h], k1[sel, hk], v1[sel, hk])
            for i in range(cu_q2[b], cu_q2[b + 1]):
                p = pos_q2[i]
                sel1 = [j for j in range(c0, c1) if duo_visible(p, 1, j - c0, 0)]
                sel2 = [j for j in range(e0, e1) if duo_visible(p, 1, pos_k2[j], 1)]
                keys = np.concatenate([k1[sel1, hk], k2[sel2, hk]], 0)
                vals = np.concatenate([v1[sel1, hk], v2[sel2, hk]], 0)
                if len(keys):
                    o2[i, h], lse2[h, i] = one_row(q2[i, h], keys, vals)
    return o1, lse1, o2, lse2


def _additive(see: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    zero = torch.zeros((), dtype=dtype)
    neg = torch.full((), torch.finfo(dtype).min, dtype=dtype)
    return torch.where(see, zero, neg)[None, None]


def duo_varlen_torch(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale):
    """Differentiable packed-varlen duo attention via the dense formulation.

    Same layout and semantics as :func:`duo_rows_f64`, computed per sequence
    with :func:`sdpa_dense` and a boolean->additive mask, so torch autograd gives
    dQ/dK/dV for both depths (depth-0 K/V collect gradient from both query
    streams, causal_cache.py:92-93 keeps them graph-attached).
    """
    nseq = len(cu_q1) - 1
    o1 = []
    o2 = []
    for b in range(nseq):
        a0, a1 = int(cu_q1[b]), int(cu_q1[b + 1])
        c0, c1 = int(cu_k1[b]), int(cu_k1[b + 1])
        d0, d1 = int(cu_q2[b]), int(cu_q2[b + 1])
        e0, e1 = int(cu_k2[b]), int(cu_k2[b + 1])
        hd = lambda x: x.transpose(0, 1)[None]  # (T,H,D) -> (1,H,T,D)
        kpos1 = torch.arange(c1 - c0)
        if a1 > a0:
            qpos1 = torch.arange(a1 - a0) + ((c1 - c0) - (a1 - a0))
            see = kpos1[None, :] <= qpos1[:, None]
            m = _additive(see, q1.dtype)
            o1.append(sdpa_dense(hd(q1[a0:a1]), hd(k1[c0:c1]), hd(v1[c0:c1]), m, scale)[0])
        if d1 > d0:
            qp = torch.as_tensor(pos_q2[d0:d1]).long()
            kp2 = torch.as_tensor(pos_k2[e0:e1]).long()
            see = torch.cat([kpos1[None, :] <= qp[:, None], kp2[None, :] <= qp[:, None]], 1)
            m = _additive(see, q1.dtype)
            K = torch.cat([k1[c0:c1], k2[e0:e1]], 0)
            V = torch.cat([v1[c0:c1], v2[e0:e1]], 0)
            o2.append(sdpa_dense(hd(q2[d0:d1]), hd(K), hd(V), m, scale)[0])
    cat = lambda xs, like: torch.cat(xs, 0) if xs else like.new_zeros((0,) + tuple(like.shape[1:]))
    return cat(o1, q1), cat(o2, q2)


# --------------------------------------------------------------------------
# Decode step against the cache (row Tq=1 of the same predicate)
# --------------------------------------------------------------------------


def duo_decode_f64(q, k1, v1, cu_k1, k2, v2, pos_k2, cu_k2, q_pos, depth, scale):
    """One query row per sequence against the packed caches, float64 numpy.

    q (nseq,Hq,D); depth[b] in {0,1}: a depth-0 query sees depth-0 keys with
    position <= q_pos[b]; a depth-1 query additionally sees depth-1 keys with
    pos_k2 <= q_pos[b].  Equals row Tq=1 of build_attention_mask + sdpa_dense.
    Returns o (nseq,Hq,D), lse (nseq,Hq).
    """
    f = lambda x: np.asarray(x, dtype=np.float64)
    q, k1, v1, k2, v2 = map(f, (q, k1, v1, k2, v2))
    nseq, Hq, D = q.shape
    g = Hq // k1.shape[1]
    o = np.zeros_like(q)
    lse = np.full((nseq, Hq), -np.inf)
    for b in range(nseq):
        c0, c1 = int(cu_k1[b]), int(cu_k1[b + 1])
        e0, e1 = int(cu_k2[b]), int(cu_k2[b + 1])
        p, d = int(q_pos[b]), int(depth[b])
        sel1 = [j for j in range(c0, c1) if duo_visible(p, d, j - c0, 0)]
        sel2 = [j for j in range(e0, e1) if duo_visible(p, d, int(pos_k2[j]), 1)]
        for h in range(Hq):
            hk = h // g
            keys = np.concatenate([k1[sel1, hk], k2[sel2, hk]], 0)
            vals = np.concatenate([v1[sel1, hk], v2[sel2, hk]], 0)
            if len(keys) == 0:
                continue
            s = keys @ q[b, h] * scale
            m = s.max()
            e = np.exp(s - m)
            o[b, h] = (e @ vals) / e.sum()
            lse[b, h] = m + np.log(e.sum())
    return o, lse


# --------------------------------------------------------------------------
# Work model shared by bench.py and the tests
# --------------------------------------------------------------------------


def visible_pairs(cu_q1, cu_k1, pos_q2, pos_k2, cu_q2, cu_k2) -> int:
    """Exact count of (query, key) pairs the mask lets through, per query head."""
    cu_q1, cu_k1, cu_q2, cu_k2 = (np.asarray(c, dtype=np.int64) for c in (cu_q1, cu_k1, cu_q2, cu_k2))
    pos_q2 = np.asarray(pos_q2, dtype=np.int64)
    pos_k2 = np.asarray(pos_k2, dtype=np.int64)
    total = 0
    for b in range(len(cu_q1) - 1):
        lq, lk = cu_q1[b + 1] - cu_q1[b], cu_k1[b + 1] - cu_k1[b]
        off = lk - lq
        qp = np.arange(lq) + off
        total += int(np.clip(qp + 1, 0, lk).sum())
        p2 = pos_q2[cu_q2[b]:cu_q2[b + 1]]
        total += int(np.clip(p2 + 1, 0, lk).sum())
        kp2 = np.sort(pos_k2[cu_k2[b]:cu_k2[b + 1]])
        total += int(np.searchsorted(kp2, p2, side="right").sum())
    return total
