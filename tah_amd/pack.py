"""Hard-token pack / scatter with the reference's call signatures.

``gather_active`` and ``scatter_back`` mirror tah/model/tah_model.py:96-176:
same arguments, same return values, same row-major packing order, same
padding.  The index work (stream compaction of the mask) and every row move run
in HIP kernels (tah_hard_index_build, tah_pad_rows_build, tah_rows_copy); torch
only allocates and fills buffers.  Floating-point tensors stay differentiable:
the backward of a row gather is a row scatter and vice versa.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops
from ._capi import TahDuoError

# True: the pack reads the number of active entries back to size its outputs exactly, the one host
# synchronisation the reference's pack has too (tah_model.py:116).  False: nothing is read back -- outputs are
# sized by upper bounds and every kernel takes the true count from device memory; ``gather_active`` then needs
# ``max_active``.  The attention callable and the cache follow the same switch.
HOST_SYNC = True


# The index of a mask is asked for several times within one model step (queries and keys of an attention call pack by
# the same valid mask; scatter_back follows gather_active with the same mask): the last few are kept, keyed by the
# mask tensor itself and its version counter, so that each mask is compacted -- and its count read back -- once.
_INDEX_MEMO: list = []
_INDEX_MEMO_SIZE = 6


class HardIndex:
    """Packed-varlen index of a (B, S) boolean mask, built on the device.

    pos[r]  position (column) of the r-th True entry in row-major order (int32)
    flat[r] its flat index b*S + s, seq[r] its row b, cu[b] entries before row b
    n, width: total count and the largest per-row count (host ints; reading them
    is the one host sync of the pack, as in tah_model.py:116).  With ``sync=False``
    nothing is read back: ``n`` and ``width`` are None, ``n_max`` = B*S bounds the
    count, ``count`` is the count on the device (one int32) and pos / flat / seq keep
    their full capacity (entries past the count are undefined).
    """

    @classmethod
    def of(cls, mask: torch.Tensor, sync: Optional[bool] = None) -> "HardIndex":
        """The index of ``mask``: the one built earlier for this very tensor (same object, not written to since, same
        read-back mode) or a new one."""
        want = HOST_SYNC if sync is None else bool(sync)
        for key, version, idx in _INDEX_MEMO:
            if key is mask and version == mask._version and idx.synced == want:
                return idx
        idx = cls(mask, sync=sync)
        _INDEX_MEMO.append((mask, mask._version, idx))
        del _INDEX_MEMO[:-_INDEX_MEMO_SIZE]
        return idx

    def __init__(self, mask: torch.Tensor, sync: Optional[bool] = None):
        if mask.dim() != 2:
            raise TahDuoError("mask must be (B, S)")
        if mask.dtype != torch.bool:
            mask = mask != 0
        self.B, self.S = mask.shape
        self.mask = mask.contiguous()
        pos, flat, seq, cu = ops.hard_index_build(self.mask)
        self.cu = cu
        self.count = cu[self.B:]
        self.n_max = self.B * self.S
        self.synced = HOST_SYNC if sync is None else sync
        if self.synced:
            cu_host = cu.cpu()
            self.n = int(cu_host[-1])
            counts = cu_host[1:] - cu_host[:-1]
            self.width = int(counts.max()) if self.B > 0 else 0
            self.pos, self.flat, self.seq = pos[: self.n], flat[: self.n], seq[: self.n]
        else:
            self.n = self.width = None
            self.pos, self.flat, self.seq = pos[: self.n_max], flat[: self.n_max], seq[: self.n_max]
        self._pad_rows: Optional[torch.Tensor] = None

    @property
    def bound(self) -> int:
        """Number of entries when known, else its upper bound (the kernels then stop at ``count``)."""
        return self.n if self.synced else self.n_max

    @property
    def n_dev(self) -> Optional[torch.Tensor]:
        return None if self.synced else self.count

    @property
    def pad_rows(self) -> torch.Tensor:
        """Row of entry r inside the right-padded (B*width) layout."""
        if self._pad_rows is None:
            self._pad_rows = ops.pad_rows_build(self.cu, self.seq, self.n, max(self.width, 1))
        return self._pad_rows

    def pad_rows_for(self, width: int, overflow: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Rows inside a right-padded (B*width) layout of a given width (entries that do not fit get -1)."""
        if self.synced and width == self.width:
            return self.pad_rows
        return ops.pad_rows_build(self.cu, self.seq, self.bound, max(width, 1), n_dev=self.n_dev, overflow=overflow)


class _RowsMove(torch.autograd.Function):
    """out = fill; out[dst_rows[r]] = src[src_rows[r]] (rows of a 2-D+ tensor flattened on dim 0)."""

    @staticmethod
    def forward(ctx, src, src_rows, dst_rows, n, out_rows, fill, dst_enable, n_dev=None):
        out = torch.full((out_rows,) + tuple(src.shape[1:]), fill, dtype=src.dtype, device=src.device)
        ops.rows_copy(src, src_rows, out, dst_rows, n, dst_enable, n_dev)
        ctx.save_for_backward(src_rows, dst_rows, dst_enable, n_dev)
        ctx.n, ctx.src_rows_total = n, src.shape[0]
        return out

    @staticmethod
    def backward(ctx, grad_out):
        src_rows, dst_rows, dst_enable, n_dev = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_src = torch.zeros((ctx.src_rows_total,) + tuple(grad_out.shape[1:]), dtype=grad_out.dtype, device=grad_out.device)
        if dst_enable is None:
            ops.rows_copy(grad_out, dst_rows, grad_src, src_rows, ctx.n, None, n_dev)
        else:
            # only enabled destination rows received data: route their gradient back, rows are unique
            en = torch.zeros(ctx.src_rows_total, dtype=torch.uint8, device=grad_out.device)
            ones = torch.ones((ctx.n, 1), dtype=torch.uint8, device=grad_out.device)
            tmp = torch.zeros((dst_enable.numel(), 1), dtype=torch.uint8, device=grad_out.device)
            ops.rows_copy(ones, None, tmp, dst_rows, ctx.n, dst_enable, n_dev)          # tmp[dst] = 1 where written
            gathered = torch.zeros((ctx.n, 1), dtype=torch.uint8, device=grad_out.device)
            ops.rows_copy(tmp, dst_rows, gathered, None, ctx.n, None, n_dev)            # per entry: was it written?
            ops.rows_copy(gathered, None, en.view(-1, 1), src_rows, ctx.n, None, n_dev)
            ops.rows_copy(grad_out, dst_rows, grad_src, src_rows, ctx.n, en, n_dev)
        return grad_src, None, None, None, None, None, None, None


def _flat_rows(t: torch.Tensor, lead: int) -> torch.Tensor:
    """(B, S, ...) -> (B*S, ...) contiguous; 2-D tensors become (B*S, 1)."""
    t = t.contiguous()
    return t.view(lead, *t.shape[2:]) if t.dim() > 2 else t.view(lead, 1)


def gather_active(current_iter_mask: torch.Tensor, *tensors, pad_value=0, max_active: Optional[int] = None
                  ) -> Tuple[Optional[torch.Tensor], ...]:
    """Pack the True positions of each row to the left (tah/model/tah_model.py:96-135).

    Returns ``(pad_mask, *gathered)``: ``pad_mask`` is (B, max_active) bool, True at
    padding; each gathered tensor is (B, max_active, ...) with pads set to
    ``pad_value``; ``None`` inputs pass through.

    ``max_active`` (not in the reference): the width of the packed block is given by the caller instead of
    being the largest row count read back from the device (tah_model.py:116) -- no host synchronisation.
    Active entries of a row beyond ``max_active`` are dropped and raise the device flag
    ``pad_mask.overflow`` (int32, one element), which the caller may check whenever it next synchronises.
    """
    dev = current_iter_mask.device
    if max_active is None and not HOST_SYNC:
        raise TahDuoError("gather_active: with tah_amd.pack.HOST_SYNC = False the packed width must be given (max_active)")
    idx = HardIndex.of(current_iter_mask, sync=max_active is None)
    B, S = idx.B, idx.S
    overflow = None
    if max_active is None:
        W, n, n_dev, pad_rows = idx.width, idx.n, None, (idx.pad_rows if idx.n else None)
    else:
        W, n, n_dev = int(max_active), idx.n_max, idx.count
        overflow = torch.zeros(1, dtype=torch.int32, device=dev)
        pad_rows = idx.pad_rows_for(W, overflow) if n else None
    pad = torch.ones((B * W, 1), dtype=torch.uint8, device=dev)
    if n:
        zeros = torch.zeros((n, 1), dtype=torch.uint8, device=dev)
        ops.rows_copy(zeros, None, pad, pad_rows, n, None, n_dev)
    pad_mask = pad.view(B, W).bool()
    if overflow is not None:
        pad_mask.overflow = overflow
    out = [pad_mask]
    for t in tensors:
        if t is None:
            out.append(None)
            continue
        if t.shape[0] != B or t.shape[1] != S:
            raise TahDuoError(f"gather_active: tensor shape {tuple(t.shape)} does not start with ({B}, {S})")
        src = _flat_rows(t, B * S)
        if n:
            g = _RowsMove.apply(src, idx.flat, pad_rows, n, B * W, pad_value, None, n_dev)
        else:
            g = torch.full((B * W,) + tuple(src.shape[1:]), pad_value, dtype=src.dtype, device=dev)
        out.append(g.view(B, W, *t.shape[2:]))
    return tuple(out)


def scatter_back(current_iter_mask: torch.Tensor, src: torch.Tensor, dest: torch.Tensor, *, in_place: bool = False,
                 assignment_mask: Optional[torch.Tensor] = None, host_sync: Optional[bool] = None) -> torch.Tensor:
    """Inverse of :func:`gather_active` (tah/model/tah_model.py:138-176).

    The valid prefix of each row of ``src`` (B, max_active, ...) is written to the
    True positions of ``current_iter_mask`` in ``dest`` (B, S, ...); with
    ``assignment_mask`` only positions where both masks are True change.  Returns
    ``dest`` itself when ``in_place`` else a new tensor.  ``host_sync=False`` (default: the module switch
    ``HOST_SYNC``): the count of active positions stays on the device; a row of ``src`` narrower than the row's
    active positions then drops the surplus instead of raising.
    """
    idx = HardIndex.of(current_iter_mask, sync=host_sync)
    B, S = idx.B, idx.S
    W = src.shape[1]
    if idx.synced and W < idx.width:
        raise TahDuoError(f"scatter_back: src has {W} columns but a row of the mask has {idx.width} active positions")
    enable = None
    if assignment_mask is not None:
        enable = (assignment_mask != 0).contiguous().view(B * S)
    needs_grad = torch.is_grad_enabled() and (src.requires_grad or dest.requires_grad)
    n, n_dev = idx.bound, idx.n_dev
    if n == 0 or W == 0:
        return dest if in_place else dest.clone()
    src_rows = idx.pad_rows_for(W)
    src_f = _flat_rows(src, B * W)
    if not needs_grad:
        out = dest if in_place else dest.clone()
        if not out.is_contiguous():
            raise TahDuoError("scatter_back: dest must be contiguous")
        ops.rows_copy(src_f, src_rows, _flat_rows(out, B * S), idx.flat, n, enable, n_dev)
        return out
    if in_place:
        raise TahDuoError("scatter_back(in_place=True) on tensors that require grad is not supported")
    # differentiable form: out = dest * keep + scatter(src)
    moved = _RowsMove.apply(src_f, src_rows, idx.flat, n, B * S, 0, enable, n_dev).view(dest.shape)
    written = torch.zeros((B * S, 1), dtype=torch.uint8, device=dest.device)
    ones = torch.ones((B * W, 1), dtype=torch.uint8, device=dest.device)
    ops.rows_copy(ones, src_rows, written, idx.flat, n, enable, n_dev)  # (entries dropped for width wrote nothing)
    keep = (written == 0).view(B, S, *([1] * (dest.dim() - 2)))
    return torch.where(keep, dest, moved)
