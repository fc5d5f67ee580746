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


class HardIndex:
    """Packed-varlen index of a (B, S) boolean mask, built on the device.

    pos[r]  position (column) of the r-th True entry in row-major order (int32)
    flat[r] its flat index b*S + s, seq[r] its row b, cu[b] entries before row b
    n, width: total count and the largest per-row count (host ints; reading them
    is the one host sync of the pack, as in tah_model.py:116).
    """

    def __init__(self, mask: torch.Tensor):
        if mask.dim() != 2:
            raise TahDuoError("mask must be (B, S)")
        if mask.dtype != torch.bool:
            mask = mask != 0
        self.B, self.S = mask.shape
        self.mask = mask.contiguous()
        pos, flat, seq, cu = ops.hard_index_build(self.mask)
        cu_host = cu.cpu()
        self.n = int(cu_host[-1])
        counts = cu_host[1:] - cu_host[:-1]
        self.width = int(counts.max()) if self.B > 0 else 0
        self.cu = cu
        self.pos, self.flat, self.seq = pos[: self.n], flat[: self.n], seq[: self.n]
        self._pad_rows: Optional[torch.Tensor] = None

    @property
    def pad_rows(self) -> torch.Tensor:
        """Row of entry r inside the right-padded (B*width) layout."""
        if self._pad_rows is None:
            self._pad_rows = ops.pad_rows_build(self.cu, self.seq, self.n, max(self.width, 1))
        return self._pad_rows


class _RowsMove(torch.autograd.Function):
    """out = fill; out[dst_rows[r]] = src[src_rows[r]] (rows of a 2-D+ tensor flattened on dim 0)."""

    @staticmethod
    def forward(ctx, src, src_rows, dst_rows, n, out_rows, fill, dst_enable):
        out = torch.full((out_rows,) + tuple(src.shape[1:]), fill, dtype=src.dtype, device=src.device)
        ops.rows_copy(src, src_rows, out, dst_rows, n, dst_enable)
        ctx.save_for_backward(src_rows, dst_rows, dst_enable)
        ctx.n, ctx.src_rows_total = n, src.shape[0]
        return out

    @staticmethod
    def backward(ctx, grad_out):
        src_rows, dst_rows, dst_enable = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        grad_src = torch.zeros((ctx.src_rows_total,) + tuple(grad_out.shape[1:]), dtype=grad_out.dtype, device=grad_out.device)
        if dst_enable is None:
            ops.rows_copy(grad_out, dst_rows, grad_src, src_rows, ctx.n)
        else:
            # only enabled destination rows received data: route their gradient back, rows are unique
            en = torch.zeros(ctx.src_rows_total, dtype=torch.uint8, device=grad_out.device)
            ones = torch.ones((ctx.n, 1), dtype=torch.uint8, device=grad_out.device)
            tmp = torch.zeros((dst_enable.numel(), 1), dtype=torch.uint8, device=grad_out.device)
            ops.rows_copy(ones, None, tmp, dst_rows, ctx.n, dst_enable)          # tmp[dst] = 1 where written
            gathered = torch.zeros((ctx.n, 1), dtype=torch.uint8, device=grad_out.device)
            ops.rows_copy(tmp, dst_rows, gathered, None, ctx.n)                  # per entry: was it written?
            ops.rows_copy(gathered, None, en.view(-1, 1), src_rows, ctx.n)
            ops.rows_copy(grad_out, dst_rows, grad_src, src_rows, ctx.n, en)
        return grad_src, None, None, None, None, None, None


def _flat_rows(t: torch.Tensor, lead: int) -> torch.Tensor:
    """(B, S, ...) -> (B*S, ...) contiguous; 2-D tensors become (B*S, 1)."""
    t = t.contiguous()
    return t.view(lead, *t.shape[2:]) if t.dim() > 2 else t.view(lead, 1)


def gather_active(current_iter_mask: torch.Tensor, *tensors, pad_value=0) -> Tuple[Optional[torch.Tensor], ...]:
    """Pack the True positions of each row to the left (tah/model/tah_model.py:96-135).

    Returns ``(pad_mask, *gathered)``: ``pad_mask`` is (B, max_active) bool, True at
    padding; each gathered tensor is (B, max_active, ...) with pads set to
    ``pad_value``; ``None`` inputs pass through.
    """
    idx = HardIndex(current_iter_mask)
    B, S, W = idx.B, idx.S, idx.width
    dev = current_iter_mask.device
    pad = torch.ones((B * W, 1), dtype=torch.uint8, device=dev)
    if idx.n:
        zeros = torch.zeros((idx.n, 1), dtype=torch.uint8, device=dev)
        ops.rows_copy(zeros, None, pad, idx.pad_rows, idx.n)
    out = [pad.view(B, W).bool()]
    for t in tensors:
        if t is None:
            out.append(None)
            continue
        if t.shape[0] != B or t.shape[1] != S:
            raise TahDuoError(f"gather_active: tensor shape {tuple(t.shape)} does not start with ({B}, {S})")
        src = _flat_rows(t, B * S)
        g = _RowsMove.apply(src, idx.flat, idx.pad_rows, idx.n, B * W, pad_value, None)
        out.append(g.view(B, W, *t.shape[2:]))
    return tuple(out)


def scatter_back(current_iter_mask: torch.Tensor, src: torch.Tensor, dest: torch.Tensor, *, in_place: bool = False,
                 assignment_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Inverse of :func:`gather_active` (tah/model/tah_model.py:138-176).

    The valid prefix of each row of ``src`` (B, max_active, ...) is written to the
    True positions of ``current_iter_mask`` in ``dest`` (B, S, ...); with
    ``assignment_mask`` only positions where both masks are True change.  Returns
    ``dest`` itself when ``in_place`` else a new tensor.
    """
    idx = HardIndex(current_iter_mask)
    B, S = idx.B, idx.S
    W = src.shape[1]
    if W < idx.width:
        raise TahDuoError(f"scatter_back: src has {W} columns but a row of the mask has {idx.width} active positions")
    enable = None
    if assignment_mask is not None:
        enable = (assignment_mask != 0).contiguous().view(B * S)
    needs_grad = torch.is_grad_enabled() and (src.requires_grad or dest.requires_grad)
    if idx.n == 0:
        return dest if in_place else dest.clone()
    src_rows = idx.pad_rows if W == idx.width else ops.pad_rows_build(idx.cu, idx.seq, idx.n, W)
    src_f = _flat_rows(src, B * W)
    if not needs_grad:
        out = dest if in_place else dest.clone()
        if not out.is_contiguous():
            raise TahDuoError("scatter_back: dest must be contiguous")
        ops.rows_copy(src_f, src_rows, _flat_rows(out, B * S), idx.flat, idx.n, enable)
        return out
    if in_place:
        raise TahDuoError("scatter_back(in_place=True) on tensors that require grad is not supported")
    # differentiable form: out = dest * keep + scatter(src)
    moved = _RowsMove.apply(src_f, src_rows, idx.flat, idx.n, B * S, 0, enable).view(dest.shape)
    written = torch.zeros((B * S, 1), dtype=torch.uint8, device=dest.device)
    ops.rows_copy(torch.ones((idx.n, 1), dtype=torch.uint8, device=dest.device), None, written, idx.flat, idx.n, enable)
    keep = (written == 0).view(B, S, *([1] * (dest.dim() - 2)))
    return torch.where(keep, dest, moved)
