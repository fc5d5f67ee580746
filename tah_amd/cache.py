"""KV cache with the read/write contract of the reference's ``TaHCache``.

Same attributes and method names as tah/model/causal_cache.py:30-239
(``current_iter_depth``, ``position_ids_to_cache``, ``valid_mask_to_cache``,
``update``, ``get_cache_upto_iter``, ``get_position_id_upto_iter``,
``get_valid_mask_upto_iter``, ``get_cache_iter_index_upto_iter``, the length
helpers, ``reorder_cache``, ``to``), so the model's forward loop drives it
unchanged.  What differs is storage and what ``update`` hands back:

* every write is kept as its own chunk per (layer, depth) -- nothing is
  concatenated on the write path (the reference re-copies the whole cache per
  layer per decode step, causal_cache.py:84-90);
* with ``enable_slabs`` the valid rows of every write are also appended, in
  place, to preallocated per-sequence slabs (tah_amd.kv_cache.KvSlabs) that the
  decode kernel streams; from the first single-token write on, the slabs are the
  only copy of K and V (the chunk lists keep positions, valid flags and lengths),
  so a long generation holds one copy of its cache and no list of tiny tensors;
* ``update`` returns the new (key, value) tensors themselves: the duo attention
  callable (tah_amd.attention.duo_attention_forward) reads the visible segments
  from the cache, so the depth-0 | depth-1 concatenation of
  causal_cache.py:101-109 is never materialised.  Set ``return_concat=True`` to
  get the reference's concatenated return value instead (compatibility / tests).
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Tuple

import torch

from ._capi import TahDuoError
from .kv_cache import KvSlabs

_Slot = Tuple[int, int]


class TaHDuoCache:
    def __init__(self, return_concat: bool = False):
        self._k: Dict[_Slot, List[torch.Tensor]] = {}
        self._v: Dict[_Slot, List[torch.Tensor]] = {}
        self._pos: Dict[_Slot, List[Optional[torch.Tensor]]] = {}
        self._valid: Dict[_Slot, List[Optional[torch.Tensor]]] = {}
        self.current_iter_depth: int = 0
        self.position_ids_to_cache: Optional[torch.Tensor] = None
        self.valid_mask_to_cache: Optional[torch.Tensor] = None
        self.batch_size: Optional[int] = None
        self.return_concat = return_concat
        self._rows: Dict[_Slot, int] = {}       # rows written per slot (pad rows included), the reference's length
        self._meta_memo: Dict[Tuple[int, int, int], Tuple[int, torch.Tensor]] = {}  # folded positions / valid flags per slot
        self._kv_dropped: Dict[_Slot, bool] = {}  # K/V of the slot live in the slabs only
        self._device: Optional[torch.device] = None
        self._dtype: Optional[torch.dtype] = None
        # native decode storage
        self._slab_cfg: Optional[Tuple[int, int]] = None
        self._slabs: Dict[_Slot, KvSlabs] = {}
        self._slab_rows: Dict[_Slot, int] = {}  # host-side upper bound on the rows any slab of the slot holds
        self._pack_memo: Dict[int, Any] = {}
        self._key_memo: Dict[Any, Any] = {}     # packed key segments of single-chunk slots, per (layer-independent) valid mask
        self._kv_packed: Dict[Any, Any] = {}    # per (layer, depth): the slot's one chunk packed, for the calls of later depths

    # ── native storage ────────────────────────────────────────────────────
    def enable_slabs(self, capacity_depth0: int, capacity_depth1: int) -> "TaHDuoCache":
        """Also keep every write in per-sequence slabs of the given row capacities (decode fast path)."""
        self._slab_cfg = (int(capacity_depth0), int(capacity_depth1))
        return self

    def slabs(self, layer_idx: int, depth: int) -> Optional[KvSlabs]:
        return self._slabs.get((layer_idx, depth))

    def _append_slabs(self, slot: _Slot, k: torch.Tensor, v: torch.Tensor, pos, valid) -> None:
        from . import ops
        from .pack import HardIndex

        B, hkv, T, d = k.shape
        sl = self._slabs.get(slot)
        if sl is None:
            sl = KvSlabs(B, self._slab_cfg[slot[1]], hkv, d, with_pos=slot[1] > 0, device=k.device, dtype=k.dtype)
            self._slabs[slot] = sl
        # A slab that is full drops rows on the device (and raises a flag nobody waits for): refuse on the
        # host instead.  Every write adds at most T rows to a sequence (T counts pad rows too, so the bound
        # is conservative); it needs no device read.
        written = self._slab_rows.get(slot, 0) + T
        if written > sl.capacity:
            raise TahDuoError(
                f"KV slabs of layer {slot[0]}, depth {slot[1]} hold {sl.capacity} rows per sequence; this write "
                f"brings a sequence to as many as {written}: enable_slabs() with a larger capacity")
        self._slab_rows[slot] = written
        if T == 1:
            # a decode step: one row per sequence, appended in place from where it lies -- rows that are not
            # valid (pad rows of the depth-1 pack) name slot -1 and are skipped; nothing is packed or read back
            key = ("step", id(valid))
            memo = self._pack_memo.get(key)
            if memo is None or memo[0] is not valid:
                rows = torch.arange(B, dtype=torch.int32, device=k.device)
                slot_of = rows if valid is None else torch.where(valid.reshape(B) != 0, rows, torch.full_like(rows, -1))
                cu1 = torch.arange(B + 1, dtype=torch.int32, device=k.device)
                memo = (valid, slot_of, cu1)
                self._pack_memo = {key: memo}
            _, slot_of, cu1 = memo
            pos_rows = pos.to(torch.int32).reshape(B).contiguous() if slot[1] > 0 else None
            sl.append(k.transpose(1, 2).reshape(B, hkv, d), v.transpose(1, 2).reshape(B, hkv, d), cu1, pos_new=pos_rows,
                      slot_of=slot_of)
            return
        # one compaction of the valid mask per forward step, shared by all layers
        key = id(valid) if valid is not None else -T
        memo = self._pack_memo.get(key)
        if memo is None or memo[0] is not valid:
            if valid is None:
                cu = torch.arange(0, (B + 1) * T, T, dtype=torch.int32, device=k.device)
                memo = (valid, None, cu, B * T, None)
            else:
                idx = HardIndex.of(valid)
                if idx.synced and idx.n == B * T:
                    memo = (valid, None, torch.arange(0, (B + 1) * T, T, dtype=torch.int32, device=k.device), B * T, None)
                else:
                    memo = (valid, idx.flat, idx.cu, idx.bound, idx.n_dev)
            self._pack_memo = {key: memo}
        _, rows, cu, n, n_dev = memo
        kt = k.transpose(1, 2).reshape(B * T, hkv, d)  # a view when k came from a (B,T,H,D) projection
        vt = v.transpose(1, 2).reshape(B * T, hkv, d)
        pos_rows = None
        if rows is not None:
            kp = torch.empty((n, hkv, d), dtype=k.dtype, device=k.device)
            vp = torch.empty((n, hkv, d), dtype=k.dtype, device=k.device)
            ops.rows_copy(kt.contiguous(), rows, kp, None, n, None, n_dev)
            ops.rows_copy(vt.contiguous(), rows, vp, None, n, None, n_dev)
            kt, vt = kp, vp
        if slot[1] > 0:
            p32 = pos.to(torch.int32).contiguous().view(B * T, 1)
            if rows is not None:
                pos_rows = torch.empty((n, 1), dtype=torch.int32, device=k.device)
                ops.rows_copy(p32, rows, pos_rows, None, n, None, n_dev)
            else:
                pos_rows = p32
            pos_rows = pos_rows.view(-1)
        if n:
            sl.append(kt, vt, cu, pos_new=pos_rows)  # (the append stops at cu[B]: n may be an upper bound)

    # ── write path (causal_cache.py:63-97) ────────────────────────────────
    def has_layer(self, layer_idx: int = 0) -> bool:
        return any(l == layer_idx for (l, _) in self._rows)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None):
        del cache_kwargs
        if self.batch_size is None:
            self.batch_size = key_states.shape[0]
        else:
            assert key_states.shape[0] == self.batch_size, (
                f"batch size mismatch: cached {self.batch_size}, got {key_states.shape[0]}")
        self._device, self._dtype = key_states.device, key_states.dtype
        if int(self.current_iter_depth) < 0:
            raise TahDuoError(f"current_iter_depth = {self.current_iter_depth}: a latent iteration depth cannot be negative")
        if int(self.current_iter_depth) > 1 and self._slab_cfg is not None:
            raise TahDuoError(f"current_iter_depth = {self.current_iter_depth}: the KV slabs of the decode path hold two latent "
                              "iterations (depth 0 and depth 1); deeper iterations run without enable_slabs()")
        slot = (layer_idx, self.current_iter_depth)
        to_slabs = self._slab_cfg is not None and not (torch.is_grad_enabled() and key_states.requires_grad)
        if to_slabs:
            self._append_slabs(slot, key_states, value_states, self.position_ids_to_cache, self.valid_mask_to_cache)
        self._rows[slot] = self._rows.get(slot, 0) + key_states.shape[-2]
        # Single-token writes that went to the slabs are not kept a second time, and what the slot kept
        # before (the prompt's chunk) is released: the decode kernel reads the slabs.
        if to_slabs and key_states.shape[-2] == 1 and not self.return_concat and self._slabs_cover(slot):
            self._kv_dropped[slot] = True
            self._k.pop(slot, None)
            self._v.pop(slot, None)
        else:
            if self._kv_dropped.get(slot):
                raise TahDuoError("this cache slot keeps K/V in its slabs only (single-token decode steps were written); "
                                  "a multi-token or differentiable write can no longer be mixed in")
            self._k.setdefault(slot, []).append(key_states)
            self._v.setdefault(slot, []).append(value_states)
        self._pos.setdefault(slot, []).append(self.position_ids_to_cache)
        self._valid.setdefault(slot, []).append(self.valid_mask_to_cache)
        if self.return_concat:
            return self.get_cache_upto_iter(layer_idx, self.current_iter_depth)
        return key_states, value_states

    def _slabs_cover(self, slot: _Slot) -> bool:
        """True when every row ever written to the slot also went to its slabs."""
        return slot in self._slabs and self._slab_rows.get(slot, 0) == self._rows.get(slot, 0)

    def has_rows(self, layer_idx: int, depth: int) -> bool:
        """Whether anything was written at (layer, depth)."""
        return self._rows.get((layer_idx, depth), 0) > 0

    # ── chunk access for the attention callable ───────────────────────────
    def chunks(self, layer_idx: int, depth: int):
        """[(k, v, pos, valid), ...] written at (layer, depth), in write order."""
        s = (layer_idx, depth)
        if self._kv_dropped.get(s):
            raise TahDuoError(f"K/V of layer {layer_idx}, depth {depth} live in the slabs only; the packed-varlen path "
                              "(multi-token queries, backward) needs a cache that kept its chunks")
        return list(zip(self._k.get(s, []), self._v.get(s, []), self._pos.get(s, []), self._valid.get(s, [])))

    # ── read views (causal_cache.py:101-158) ──────────────────────────────
    def get_cache_upto_iter(self, layer_idx: int, upto_iter_idx: int):
        if any(self._kv_dropped.get((layer_idx, d)) for d in range(upto_iter_idx + 1)):
            raise TahDuoError("get_cache_upto_iter: K/V of this layer live in the slabs only (decode steps were "
                              "written with enable_slabs); construct the cache with return_concat=True to keep them")
        ks = [t for d in range(upto_iter_idx + 1) for t in self._k.get((layer_idx, d), [])]
        if not ks:
            return None, None
        vs = [t for d in range(upto_iter_idx + 1) for t in self._v.get((layer_idx, d), [])]
        return (ks[0], vs[0]) if len(ks) == 1 else (torch.cat(ks, dim=-2), torch.cat(vs, dim=-2))

    def _meta_upto_iter(self, store, layer_idx: int, upto_iter_idx: int, init_batch_size: int) -> torch.Tensor:
        parts = []
        for d in range(upto_iter_idx + 1):
            ts = store.get((layer_idx, d), [])
            if len(ts) > 1 and all(t is not None for t in ts):
                # The per-step pieces are folded in a memo of their own (a long generation stays cheap: one
                # concatenation of the folded part and the new pieces per call).  The lists themselves stay one
                # entry per write: chunks() pairs them with the K/V chunks entry by entry.
                key = (id(store), layer_idx, d)
                n, folded = self._meta_memo.get(key, (0, None))
                if n != len(ts):
                    folded = torch.cat(([folded] if n else []) + ts[n:], dim=-1) if n < len(ts) else torch.cat(ts, dim=-1)
                    self._meta_memo[key] = (len(ts), folded)
                ts = [folded]
            parts += ts
        if not parts:
            return torch.empty((init_batch_size, 0), device=self.device, dtype=torch.long)
        return parts[0] if len(parts) == 1 else torch.cat(parts, dim=-1)

    def get_position_id_upto_iter(self, layer_idx: int, upto_iter_idx: int, init_batch_size: int = 1) -> torch.Tensor:
        return self._meta_upto_iter(self._pos, layer_idx, upto_iter_idx, init_batch_size)

    def get_valid_mask_upto_iter(self, layer_idx: int, upto_iter_idx: int, init_batch_size: int = 1) -> torch.Tensor:
        return self._meta_upto_iter(self._valid, layer_idx, upto_iter_idx, init_batch_size)

    def get_cache_iter_index_upto_iter(self, layer_idx: int, upto_iter_idx: int) -> torch.Tensor:
        lens = [self.get_cache_length(layer_idx, d) for d in range(upto_iter_idx + 1)]
        if sum(lens) == 0:
            return torch.empty((0,), device=self.device, dtype=torch.long)
        return torch.cat([torch.full((n,), d, device=self.device, dtype=torch.long) for d, n in enumerate(lens) if n > 0])

    # ── lengths & misc protocol (causal_cache.py:162-205) ─────────────────
    def get_cache_length(self, layer_idx: Optional[int] = 0, iter_idx: Optional[int] = None) -> int:
        return sum(n for (l, d), n in self._rows.items() if l == layer_idx and (iter_idx is None or d == iter_idx))

    def get_kv_length_upto_iter(self, layer_idx: int = 0, upto_iter_idx: int = 0) -> int:
        return sum(self.get_cache_length(layer_idx, d) for d in range(upto_iter_idx + 1))

    def get_seq_length(self, layer_idx: Optional[int] = 0, iter_idx: Optional[int] = 0) -> int:
        return self.get_cache_length(layer_idx, iter_idx)

    def get_usable_length(self, new_seq_length: int, layer_idx: Optional[int] = 0) -> int:
        del new_seq_length
        return self.get_cache_length(layer_idx)

    def get_max_length(self) -> Optional[int]:
        return None

    def get_max_cache_shape(self) -> Optional[int]:
        return None

    def get_mask_sizes(self, cache_position: torch.Tensor, layer_idx: int) -> Tuple[int, int]:
        return cache_position.shape[0] + self.get_cache_length(layer_idx), 0

    def reorder_cache(self, beam_idx: torch.LongTensor) -> None:
        """Batch row i continues from row beam_idx[i] (causal_cache.py:201-205: K and V only, the staged positions
        and valid flags of the chunks stay as they are).  Slabs move their rows, positions and lengths together."""
        for store in (self._k, self._v):
            for slot, ts in store.items():
                store[slot] = [t.index_select(0, beam_idx.to(t.device)) for t in ts]
        for sl in self._slabs.values():
            sl.reorder(beam_idx)

    # ── device / dtype (causal_cache.py:209-239) ──────────────────────────
    @property
    def device(self) -> torch.device:
        for ts in self._k.values():
            return ts[0].device
        return self._device if self._device is not None else torch.device("cpu")

    @property
    def dtype(self) -> torch.dtype:
        for ts in self._k.values():
            return ts[0].dtype
        return self._dtype if self._dtype is not None else torch.bfloat16

    def to(self, *args, **kwargs) -> "TaHDuoCache":
        device, dtype = kwargs.get("device"), kwargs.get("dtype")
        for arg in args:
            if isinstance(arg, (torch.device, str)):
                device = arg
            elif isinstance(arg, torch.dtype):
                dtype = arg
        if device is not None:
            self._device = torch.device(device)
        if dtype is not None:
            self._dtype = dtype
        if self._slabs and (device is not None or dtype is not None):
            raise TahDuoError("cannot move a cache whose slabs are already allocated")
        mv = lambda t, with_dtype: t if t is None else t.to(**({"device": device} if device is not None else {}),
                                                            **({"dtype": dtype} if dtype is not None and with_dtype else {}))
        self._meta_memo.clear()
        for store, with_dtype in ((self._k, True), (self._v, True), (self._pos, False), (self._valid, False)):
            for slot, ts in store.items():
                store[slot] = [mv(t, with_dtype) for t in ts]
        return self

    def __len__(self) -> int:
        return len({l for (l, _) in self._rows})
