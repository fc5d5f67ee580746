"""Native per-layer KV storage for the duo-causal decode path.

One :class:`KvSlabs` holds one depth (iteration) of one decoder layer: a slab
of ``capacity`` rows per sequence slot, head-major inside the slab
(``[slot, Hkv, capacity, D]``), so that the decode kernel streams each
(sequence, kv head) as one contiguous run.  Lengths live on the device; appends
and reads never synchronise with the host.  This replaces the growing
``torch.cat`` tensors of the reference cache (tah/model/causal_cache.py:84-95).
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import _capi, _lib
from .ops import _dev_check, _i32, _ptr, _stream, _thd


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

    def segment(self) -> _capi.KvSegment:
        s = _capi.KvSegment()
        s.k, s.v = self.k.data_ptr(), self.v.data_ptr()
        s.pos = None if self.pos is None else self.pos.data_ptr()
        s.start, s.len = self.start.data_ptr(), self.len.data_ptr()
        s.k_row_stride = s.v_row_stride = self.d
        s.k_head_stride = s.v_head_stride = self.capacity * self.d
        s.capacity, s.nslots = self.capacity, self.nslots
        return s

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
        """Append rows [cu_new[i], cu_new[i+1]) of k_new/v_new ([rows, Hkv, D]) to slot slot_of[i] (default i)."""
        lib = _lib.lib()
        _thd(k_new, "k_new"), _thd(v_new, "v_new"), _i32(cu_new, "cu_new")
        _dev_check(k_new, v_new, cu_new, pos_new, slot_of, self.k)
        if (pos_new is None) != (self.pos is None):
            raise _capi.TahDuoError("pos_new must be given exactly for slabs created with_pos=True")
        a = _capi.KvAppendArgs()
        a.k_new, a.v_new, a.pos_new = _ptr(k_new), _ptr(v_new), _ptr(pos_new)
        a.k_row_stride, a.k_head_stride = k_new.stride(0), k_new.stride(1)
        a.v_row_stride, a.v_head_stride = v_new.stride(0), v_new.stride(1)
        a.cu_new, a.slot_of = cu_new.data_ptr(), _ptr(slot_of)
        a.nseq, a.total_new, a.hkv, a.d = cu_new.numel() - 1, k_new.shape[0], self.hkv, self.d
        a.cache = self.segment()
        a.overflow = self.overflow.data_ptr()
        _capi.check(lib, lib.tah_kv_append(ctypes.byref(a), _stream(self.k)), "tah_kv_append")


def qk_norm_rope(q: torch.Tensor, k: torch.Tensor, q_weight: torch.Tensor, k_weight: torch.Tensor,
                 cos: torch.Tensor, sin: torch.Tensor, eps: float, *, v: Optional[torch.Tensor] = None,
                 cache: Optional[KvSlabs] = None, cu_new: Optional[torch.Tensor] = None,
                 pos_new: Optional[torch.Tensor] = None, slot_of: Optional[torch.Tensor] = None,
                 in_place: bool = False, one_row_per_seq: bool = False):
    """Per-head RMSNorm of q and k, rotary embedding of both and, with ``cache``, the KV append, in one
    kernel: the steps of ``Qwen3Attention.forward`` between the projections and the attention call
    (``q_norm``, ``k_norm``, ``apply_rotary_pos_emb``, ``past_key_values.update``), with bf16 roundings
    where the eager modules round.

    q ``[rows, Hq, 128]``, k / v ``[rows, Hkv, 128]`` (token-major, as the projections produce them),
    weights ``[128]``, cos / sin ``[rows, 128]``, all bf16.  Returns ``(q_out, k_out)``; with ``cache``
    K and V go to the slabs (rows ``[cu_new[i], cu_new[i+1])`` to slot ``slot_of[i]``) and ``k_out`` is
    ``None``.  ``one_row_per_seq=True`` (a decode step: every sequence brings at most one row, all slots
    different) lets the same launch advance the slab lengths."""
    lib = _lib.lib()
    _thd(q, "q"), _thd(k, "k")
    _dev_check(q, k, v, q_weight, k_weight, cos, sin, cu_new, pos_new, slot_of, cache.k if cache is not None else None)
    for t, name in ((q_weight, "q_weight"), (k_weight, "k_weight")):
        if t.dtype != torch.bfloat16 or t.shape != (q.shape[2],) or not t.is_contiguous():
            raise _capi.TahDuoError(f"{name} must be a contiguous bf16 [{q.shape[2]}] tensor")
    for t, name in ((cos, "cos"), (sin, "sin")):
        if t.dtype != torch.bfloat16 or t.shape != (q.shape[0], q.shape[2]) or t.stride(1) != 1:
            raise _capi.TahDuoError(f"{name} must be a bf16 [rows, {q.shape[2]}] tensor with unit inner stride")
    if cos.stride(0) != sin.stride(0):
        raise _capi.TahDuoError("cos and sin must share their row stride")
    if k.shape[0] != q.shape[0]:
        raise _capi.TahDuoError("q and k must have one row per token")
    a = _capi.QkPrepArgs()
    q_out = q if in_place else torch.empty_like(q)
    a.q, a.k, a.v, a.q_out = _ptr(q), _ptr(k), _ptr(v), _ptr(q_out)
    a.q_row_stride, a.q_head_stride = q.stride(0), q.stride(1)
    a.k_row_stride, a.k_head_stride = k.stride(0), k.stride(1)
    a.q_out_row_stride, a.q_out_head_stride = q_out.stride(0), q_out.stride(1)
    if v is not None:
        _thd(v, "v")
        a.v_row_stride, a.v_head_stride = v.stride(0), v.stride(1)
    a.q_weight, a.k_weight, a.cos, a.sin = _ptr(q_weight), _ptr(k_weight), _ptr(cos), _ptr(sin)
    a.cos_sin_row_stride = cos.stride(0)
    a.eps = float(eps)
    a.rows, a.hq, a.hkv, a.d = q.shape[0], q.shape[1], k.shape[1], q.shape[2]
    k_out = None
    if cache is not None:
        if v is None or cu_new is None:
            raise _capi.TahDuoError("appending needs v and cu_new")
        if (pos_new is None) != (cache.pos is None):
            raise _capi.TahDuoError("pos_new must be given exactly for slabs created with_pos=True")
        _i32(cu_new, "cu_new")
        a.append = 1
        a.append_one_row_per_seq = 1 if one_row_per_seq else 0
        a.cu_new, a.slot_of, a.pos_new = cu_new.data_ptr(), _ptr(slot_of), _ptr(pos_new)
        a.nseq = cu_new.numel() - 1
        a.cache = cache.segment()
        a.overflow = cache.overflow.data_ptr()
    else:
        k_out = k if in_place else torch.empty_like(k)
        a.k_out = _ptr(k_out)
        a.k_out_row_stride, a.k_out_head_stride = k_out.stride(0), k_out.stride(1)
    _capi.check(lib, lib.tah_qk_prep(ctypes.byref(a), _stream(q)), "tah_qk_prep")
    return q_out, k_out


_WORKSPACES = {}


def decode(q: torch.Tensor, q_slot: torch.Tensor, q_pos: torch.Tensor, c1: KvSlabs, c2: Optional[KvSlabs], *,
           scale: float, depth: int = 0, q_depth: Optional[torch.Tensor] = None, return_lse: bool = False,
           out: Optional[torch.Tensor] = None, lse_out: Optional[torch.Tensor] = None, static_scratch: bool = False):
    """One decode step: q [nq, Hq, D] bf16, one row per (sequence, depth) being decoded.

    Row i belongs to cache slot q_slot[i], sits at position q_pos[i], and sees the
    depth-0 rows with index <= q_pos[i] plus, at depth 1, the depth-1 rows with
    pos <= q_pos[i].  ``q_depth`` (int32 [nq]) overrides ``depth`` per row.
    ``out`` / ``lse_out`` take the results when given.  ``static_scratch=True`` calls
    ``tah_duo_decode_static``: the split-K partials go to the buffer the library holds on the GPU, so with
    ``out`` given the call allocates nothing (callers under graph capture); requests beyond
    ``_capi.STATIC_SCRATCH_BYTES`` raise.
    """
    lib = _lib.lib()
    _thd(q, "q"), _i32(q_slot, "q_slot"), _i32(q_pos, "q_pos")
    _dev_check(q, q_slot, q_pos, q_depth, c1.k)
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
        nbytes = lib.tah_duo_decode_workspace_bytes(nq, hq, c1.capacity, c2.capacity if need2 else 0)
        key = (q.device, _stream(q))
        ws = _WORKSPACES.get(key)
        if ws is None or ws.numel() < nbytes:
            ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=q.device)
            _WORKSPACES[key] = ws
    a = _capi.DuoDecodeArgs()
    a.q, a.o, a.lse = _ptr(q), _ptr(o), _ptr(lse)
    a.q_row_stride, a.q_head_stride, a.o_row_stride, a.o_head_stride = q.stride(0), q.stride(1), o.stride(0), o.stride(1)
    a.q_slot, a.q_pos, a.q_depth = q_slot.data_ptr(), q_pos.data_ptr(), _ptr(q_depth)
    a.depth = depth
    a.c1 = c1.segment()
    if need2:
        a.c2 = c2.segment()
    a.nq, a.hq, a.hkv, a.d, a.scale = nq, hq, c1.hkv, d, float(scale)
    if static_scratch:
        _capi.check(lib, lib.tah_duo_decode_static(ctypes.byref(a), _stream(q)), "tah_duo_decode_static")
    else:
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
        _capi.check(lib, lib.tah_duo_decode(ctypes.byref(a), _stream(q)), "tah_duo_decode")
    return (o, lse) if return_lse else o
