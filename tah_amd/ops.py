"""Thin torch-facing wrappers over the C ABI (include/tah_duo.h).

Every function here hands raw device pointers, sizes and the current HIP stream
to libtah_duo.so.  Nothing is computed in Python or by torch operators: torch
only owns the memory.
"""
from __future__ import annotations

import ctypes
from typing import Optional, Tuple

import torch

from . import _capi, _lib

# Set only by the CPU-execution tests, which bind the same prototypes to a host
# build of the kernels; the product never touches it.
_HOST_POINTERS_OK = False


def _stream(t: torch.Tensor) -> int:
    if t.is_cuda:
        return torch.cuda.current_stream(t.device).cuda_stream
    return 0


def _dev_check(*ts: Optional[torch.Tensor]) -> None:
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda and not _HOST_POINTERS_OK:
            raise _capi.TahDuoError("tah_amd ops need CUDA/HIP tensors (no CPU path exists)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise _capi.TahDuoError(f"tensors on different devices: {dev} vs {t.device}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None or t.numel() == 0 else t.data_ptr()


def _i32(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise _capi.TahDuoError(f"{name} must be a contiguous int32 tensor")
    return t


def _thd(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dim() != 3 or t.dtype != torch.bfloat16:
        raise _capi.TahDuoError(f"{name} must be a bf16 [rows, heads, head_dim] tensor, got {t.dtype} {tuple(t.shape)}")
    if t.numel() and t.stride(2) != 1:
        raise _capi.TahDuoError(f"{name}: head_dim must be contiguous")
    return t


def _fill_stream(s: _capi.DuoStream, q, k, v, o, lse, cu_q, cu_k, pos_q, pos_k) -> None:
    s.q, s.k, s.v, s.o, s.lse = _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse)
    s.cu_q, s.cu_k = cu_q.data_ptr(), cu_k.data_ptr()
    s.pos_q, s.pos_k = _ptr(pos_q), _ptr(pos_k)
    s.q_row_stride, s.q_head_stride = q.stride(0), q.stride(1)
    s.k_row_stride, s.k_head_stride = k.stride(0), k.stride(1)
    s.v_row_stride, s.v_head_stride = v.stride(0), v.stride(1)
    s.o_row_stride, s.o_head_stride = o.stride(0), o.stride(1)
    s.total_q, s.total_k = q.shape[0], k.shape[0]


def duo_fwd_varlen(q1, k1, v1, cu_q1, cu_k1, q2, k2, v2, pos_q2, pos_k2, cu_q2, cu_k2, scale: float
                   ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Duo-causal attention forward on packed varlen bf16 tensors.

    q1 [T1q,Hq,D], k1/v1 [T1k,Hkv,D], cu_q1/cu_k1 int32 [nseq+1]: depth-0 stream.
    q2 [T2q,Hq,D], k2/v2 [T2k,Hkv,D], pos_q2/pos_k2 int32, cu_q2/cu_k2: depth-1 stream
    (hard tokens).  Returns o1, lse1 [Hq,T1q], o2, lse2 [Hq,T2q].
    """
    lib = _lib.lib()
    for n, t in (("q1", q1), ("k1", k1), ("v1", v1), ("q2", q2), ("k2", k2), ("v2", v2)):
        _thd(t, n)
    for n, t in (("cu_q1", cu_q1), ("cu_k1", cu_k1), ("cu_q2", cu_q2), ("cu_k2", cu_k2),
                 ("pos_q2", pos_q2), ("pos_k2", pos_k2)):
        _i32(t, n)
    _dev_check(q1, k1, v1, q2, k2, v2, cu_q1, cu_k1, cu_q2, cu_k2, pos_q2, pos_k2)
    nseq = cu_q1.numel() - 1
    if not (cu_k1.numel() == cu_q2.numel() == cu_k2.numel() == nseq + 1):
        raise _capi.TahDuoError("cu_seqlens tensors must all have nseq+1 entries")
    if pos_q2.numel() != q2.shape[0] or pos_k2.numel() != k2.shape[0] or k1.shape != v1.shape or k2.shape != v2.shape:
        raise _capi.TahDuoError("inconsistent row counts")
    hq, d = q1.shape[1], q1.shape[2]
    hkv = k1.shape[1]
    o1 = torch.empty((q1.shape[0], hq, d), dtype=q1.dtype, device=q1.device)
    o2 = torch.empty((q2.shape[0], hq, d), dtype=q1.dtype, device=q1.device)
    lse1 = torch.empty((hq, q1.shape[0]), dtype=torch.float32, device=q1.device)
    lse2 = torch.empty((hq, q2.shape[0]), dtype=torch.float32, device=q1.device)
    a = _capi.DuoFwdArgs()
    _fill_stream(a.s1, q1, k1, v1, o1, lse1, cu_q1, cu_k1, None, None)
    _fill_stream(a.s2, q2, k2, v2, o2, lse2, cu_q2, cu_k2, pos_q2, pos_k2)
    a.nseq, a.hq, a.hkv, a.d, a.scale = nseq, hq, hkv, d, float(scale)
    _capi.check(lib, lib.tah_duo_fwd_varlen(ctypes.byref(a), _stream(q1)), "tah_duo_fwd_varlen")
    return o1, lse1, o2, lse2


def _fill_bwd_stream(g: _capi.DuoBwdStream, d_o, dq, dk, dv, delta) -> None:
    g.d_o, g.dq, g.dk, g.dv, g.delta = _ptr(d_o), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(delta)
    g.do_row_stride, g.do_head_stride = d_o.stride(0), d_o.stride(1)
    g.dq_row_stride, g.dq_head_stride = dq.stride(0), dq.stride(1)
    g.dk_row_stride, g.dk_head_stride = dk.stride(0), dk.stride(1)
    g.dv_row_stride, g.dv_head_stride = dv.stride(0), dv.stride(1)


def duo_bwd_varlen(q1, k1, v1, o1, lse1, do1, cu_q1, cu_k1, q2, k2, v2, o2, lse2, do2, pos_q2, pos_k2, cu_q2, cu_k2,
                   scale: float):
    """Backward of :func:`duo_fwd_varlen`; returns dq1, dk1, dv1, dq2, dk2, dv2 (bf16)."""
    lib = _lib.lib()
    for n, t in (("q1", q1), ("k1", k1), ("v1", v1), ("o1", o1), ("do1", do1),
                 ("q2", q2), ("k2", k2), ("v2", v2), ("o2", o2), ("do2", do2)):
        _thd(t, n)
    for n, t in (("cu_q1", cu_q1), ("cu_k1", cu_k1), ("cu_q2", cu_q2), ("cu_k2", cu_k2),
                 ("pos_q2", pos_q2), ("pos_k2", pos_k2)):
        _i32(t, n)
    _dev_check(q1, k1, v1, o1, lse1, do1, q2, k2, v2, o2, lse2, do2, cu_q1, cu_k1, cu_q2, cu_k2, pos_q2, pos_k2)
    if do1.shape != q1.shape or do2.shape != q2.shape or o1.shape != q1.shape or o2.shape != q2.shape:
        raise _capi.TahDuoError("o / dO shapes must match q")
    if lse1.dtype != torch.float32 or lse2.dtype != torch.float32 or not lse1.is_contiguous() or not lse2.is_contiguous():
        raise _capi.TahDuoError("lse must be contiguous float32 [Hq, rows]")
    nseq = cu_q1.numel() - 1
    hq, d = q1.shape[1], q1.shape[2]
    dq1, dk1, dv1 = torch.empty_like(q1, memory_format=torch.contiguous_format), torch.empty(k1.shape, dtype=k1.dtype, device=k1.device), torch.empty(v1.shape, dtype=v1.dtype, device=v1.device)
    dq2, dk2, dv2 = torch.empty_like(q2, memory_format=torch.contiguous_format), torch.empty(k2.shape, dtype=k2.dtype, device=k2.device), torch.empty(v2.shape, dtype=v2.dtype, device=v2.device)
    delta1 = torch.empty((hq, q1.shape[0]), dtype=torch.float32, device=q1.device)
    delta2 = torch.empty((hq, q2.shape[0]), dtype=torch.float32, device=q1.device)
    a = _capi.DuoBwdArgs()
    _fill_stream(a.fwd.s1, q1, k1, v1, o1, lse1, cu_q1, cu_k1, None, None)
    _fill_stream(a.fwd.s2, q2, k2, v2, o2, lse2, cu_q2, cu_k2, pos_q2, pos_k2)
    a.fwd.nseq, a.fwd.hq, a.fwd.hkv, a.fwd.d, a.fwd.scale = nseq, hq, k1.shape[1], d, float(scale)
    _fill_bwd_stream(a.g1, do1, dq1, dk1, dv1, delta1)
    _fill_bwd_stream(a.g2, do2, dq2, dk2, dv2, delta2)
    _capi.check(lib, lib.tah_duo_bwd_varlen(ctypes.byref(a), _stream(q1)), "tah_duo_bwd_varlen")
    return dq1, dk1, dv1, dq2, dk2, dv2


def _fill_mask(m: _capi.AdditiveMask, mask: torch.Tensor, nseq: int, hq: int, tq: int, tk: int) -> None:
    """mask (B or 1, Hq or 1, Tq, Tkv) additive, bf16 or float32; broadcast dims get stride 0."""
    if mask.dim() != 4 or mask.dtype not in (torch.bfloat16, torch.float32):
        raise _capi.TahDuoError("additive mask must be a 4-D bf16 or float32 tensor (B|1, Hq|1, Tq, Tkv)")
    if mask.shape[0] not in (1, nseq) or mask.shape[1] not in (1, hq) or mask.shape[2] != tq or mask.shape[3] != tk:
        raise _capi.TahDuoError(f"additive mask shape {tuple(mask.shape)} does not match (B={nseq}, Hq={hq}, Tq={tq}, Tkv={tk})")
    m.mask = mask.data_ptr()
    m.seq_stride = mask.stride(0) if mask.shape[0] != 1 else 0
    m.head_stride = mask.stride(1) if mask.shape[1] != 1 else 0
    m.q_stride, m.k_stride = mask.stride(2), mask.stride(3)
    m.dtype = 1 if mask.dtype == torch.float32 else 0


def _dense_cu(q: torch.Tensor, nseq: int, t: int) -> torch.Tensor:
    return torch.arange(0, (nseq + 1) * t, t, dtype=torch.int32, device=q.device)


def duo_fwd_masked(q, k, v, mask, nseq: int, scale: float):
    """Compatibility mode: ``softmax(q k^T * scale + mask) v`` with a dense additive mask.

    q [B*Tq,Hq,D], k/v [B*Tkv,Hkv,D] (batch rows one after another), mask (B|1, Hq|1, Tq, Tkv).
    Returns o [B*Tq,Hq,D] and lse [Hq, B*Tq].
    """
    lib = _lib.lib()
    for n, t in (("q", q), ("k", k), ("v", v)):
        _thd(t, n)
    _dev_check(q, k, v, mask)
    if nseq <= 0 or q.shape[0] % nseq or k.shape[0] % nseq or k.shape != v.shape:
        raise _capi.TahDuoError("row counts must be multiples of the batch size")
    tq, tk = q.shape[0] // nseq, k.shape[0] // nseq
    hq, d = q.shape[1], q.shape[2]
    o = torch.empty((q.shape[0], hq, d), dtype=q.dtype, device=q.device)
    lse = torch.empty((hq, q.shape[0]), dtype=torch.float32, device=q.device)
    cu_q, cu_k = _dense_cu(q, nseq, tq), _dense_cu(q, nseq, tk)
    zc = torch.zeros(nseq + 1, dtype=torch.int32, device=q.device)
    e = q[:0]
    a = _capi.DuoFwdArgs()
    _fill_stream(a.s1, q, k, v, o, lse, cu_q, cu_k, None, None)
    _fill_stream(a.s2, e, k[:0], v[:0], e, lse[:, :0], zc, zc, None, None)
    a.nseq, a.hq, a.hkv, a.d, a.scale = nseq, hq, k.shape[1], d, float(scale)
    m = _capi.AdditiveMask()
    _fill_mask(m, mask, nseq, hq, tq, tk)
    _capi.check(lib, lib.tah_duo_fwd_masked(ctypes.byref(a), ctypes.byref(m), _stream(q)), "tah_duo_fwd_masked")
    return o, lse


def duo_bwd_masked(q, k, v, o, lse, d_o, mask, nseq: int, scale: float):
    """Backward of :func:`duo_fwd_masked`; returns dq, dk, dv (bf16)."""
    lib = _lib.lib()
    for n, t in (("q", q), ("k", k), ("v", v), ("o", o), ("d_o", d_o)):
        _thd(t, n)
    _dev_check(q, k, v, o, lse, d_o, mask)
    if d_o.shape != q.shape or o.shape != q.shape:
        raise _capi.TahDuoError("o / dO shapes must match q")
    if lse.dtype != torch.float32 or not lse.is_contiguous():
        raise _capi.TahDuoError("lse must be contiguous float32 [Hq, rows]")
    tq, tk = q.shape[0] // nseq, k.shape[0] // nseq
    hq, d = q.shape[1], q.shape[2]
    dq = torch.empty_like(q, memory_format=torch.contiguous_format)
    dk = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    dv = torch.empty(v.shape, dtype=v.dtype, device=v.device)
    delta = torch.empty((hq, q.shape[0]), dtype=torch.float32, device=q.device)
    cu_q, cu_k = _dense_cu(q, nseq, tq), _dense_cu(q, nseq, tk)
    zc = torch.zeros(nseq + 1, dtype=torch.int32, device=q.device)
    e = q[:0]
    a = _capi.DuoBwdArgs()
    _fill_stream(a.fwd.s1, q, k, v, o, lse, cu_q, cu_k, None, None)
    _fill_stream(a.fwd.s2, e, k[:0], v[:0], e, lse[:, :0], zc, zc, None, None)
    a.fwd.nseq, a.fwd.hq, a.fwd.hkv, a.fwd.d, a.fwd.scale = nseq, hq, k.shape[1], d, float(scale)
    _fill_bwd_stream(a.g1, d_o, dq, dk, dv, delta)
    _fill_bwd_stream(a.g2, e, e, k[:0], v[:0], delta[:, :0])
    m = _capi.AdditiveMask()
    _fill_mask(m, mask, nseq, hq, tq, tk)
    _capi.check(lib, lib.tah_duo_bwd_masked(ctypes.byref(a), ctypes.byref(m), _stream(q)), "tah_duo_bwd_masked")
    return dq, dk, dv


def hard_index_build(mask: torch.Tensor):
    """(B, S) bool/uint8 mask -> pos int32 [B*S cap], flat int32, seq int32, cu int32 [B+1].

    Only the first cu[B] entries of pos/flat/seq are defined.  No host sync.
    """
    lib = _lib.lib()
    _dev_check(mask)
    if mask.dim() != 2 or mask.dtype not in (torch.bool, torch.uint8):
        raise _capi.TahDuoError("mask must be a (B, S) bool or uint8 tensor")
    m = mask.contiguous()
    B, S = m.shape
    cap = max(B * S, 1)
    pos = torch.empty(cap, dtype=torch.int32, device=m.device)
    flat = torch.empty(cap, dtype=torch.int32, device=m.device)
    seq = torch.empty(cap, dtype=torch.int32, device=m.device)
    cu = torch.empty(B + 1, dtype=torch.int32, device=m.device)
    _capi.check(lib, lib.tah_hard_index_build(_ptr(m), B, S, pos.data_ptr(), flat.data_ptr(), seq.data_ptr(),
                                              cu.data_ptr(), _stream(m)), "tah_hard_index_build")
    return pos, flat, seq, cu


def pad_rows_build(cu: torch.Tensor, seq_of: torch.Tensor, n: int, width: int, n_dev: Optional[torch.Tensor] = None,
                   overflow: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of the packed entries inside the right-padded (B, width) layout.  ``n_dev`` (device int32, one
    element): only the first ``min(n, n_dev)`` entries are defined -- ``n`` may then be an upper bound."""
    lib = _lib.lib()
    _dev_check(cu, seq_of, n_dev, overflow)
    out = torch.empty(max(n, 1), dtype=torch.int32, device=cu.device)
    _capi.check(lib, lib.tah_pad_rows_build(cu.data_ptr(), seq_of.data_ptr(), n, _ptr(n_dev), width, out.data_ptr(),
                                            _ptr(overflow), _stream(cu)), "tah_pad_rows_build")
    return out[:n]


def rows_copy(src: torch.Tensor, src_rows: Optional[torch.Tensor], dst: torch.Tensor,
              dst_rows: Optional[torch.Tensor], n: int, dst_enable: Optional[torch.Tensor] = None,
              n_dev: Optional[torch.Tensor] = None) -> None:
    """dst[dst_rows[r]] = src[src_rows[r]] for r < n; src/dst are [rows, ...] with contiguous rows.

    dst_enable (bool/uint8, one entry per row of dst): rows whose entry is 0 are left untouched.
    n_dev (device int32, one element): entries r >= n_dev are skipped too, so ``n`` may be an upper bound
    and the true count never has to reach the host.
    """
    lib = _lib.lib()
    _dev_check(src, dst, src_rows, dst_rows, dst_enable, n_dev)
    if dst_enable is not None and (dst_enable.dtype not in (torch.bool, torch.uint8) or not dst_enable.is_contiguous()
                                   or dst_enable.numel() != dst.shape[0]):
        raise _capi.TahDuoError("rows_copy: dst_enable must be a contiguous bool/uint8 tensor with one entry per dst row")
    if n == 0:
        return
    if src.dtype != dst.dtype or src.shape[1:] != dst.shape[1:]:
        raise _capi.TahDuoError("rows_copy: src and dst rows differ in dtype or shape")
    for t in (src, dst):
        if not t[0].is_contiguous():
            raise _capi.TahDuoError("rows_copy: rows must be contiguous")
    row_bytes = src[0].numel() * src.element_size()
    sstride = (src.stride(0) if src.shape[0] > 1 else src[0].numel()) * src.element_size()
    dstride = (dst.stride(0) if dst.shape[0] > 1 else dst[0].numel()) * dst.element_size()
    _capi.check(lib, lib.tah_rows_copy(src.data_ptr(), _ptr(src_rows), dst.data_ptr(), _ptr(dst_rows), _ptr(dst_enable), n,
                                       _ptr(n_dev), row_bytes, sstride, dstride, _stream(src)), "tah_rows_copy")


def topk_mix(logits: torch.Tensor, embedding: torch.Tensor, topk: int, row_enable: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Soft input embedding of hard tokens (tah_model.py:57-75): logits bf16 [rows, V] -> bf16 [rows, H], the
    softmax over each row's top-k logits times the matching rows of ``embedding`` [V, H].  ``row_enable``
    (bool/uint8 [rows]): rows with 0 are skipped and keep what ``out`` held."""
    lib = _lib.lib()
    _dev_check(logits, embedding, row_enable, out)
    if logits.dim() != 2 or embedding.dim() != 2 or logits.dtype != torch.bfloat16 or embedding.dtype != torch.bfloat16:
        raise _capi.TahDuoError("topk_mix: logits [rows, V] and embedding [V, H] must be bf16")
    if logits.shape[1] != embedding.shape[0] or logits.stride(1) != 1 or embedding.stride(1) != 1:
        raise _capi.TahDuoError("topk_mix: vocabulary sizes differ or the inner dimension is not contiguous")
    rows, H = logits.shape[0], embedding.shape[1]
    if out is None:
        out = torch.zeros((rows, H), dtype=embedding.dtype, device=logits.device) if row_enable is not None else \
            torch.empty((rows, H), dtype=embedding.dtype, device=logits.device)
    if out.shape != (rows, H) or out.dtype != embedding.dtype or out.stride(1) != 1:
        raise _capi.TahDuoError("topk_mix: out must be bf16 [rows, H]")
    if row_enable is not None and (row_enable.dtype not in (torch.bool, torch.uint8) or row_enable.numel() != rows
                                   or not row_enable.is_contiguous()):
        raise _capi.TahDuoError("topk_mix: row_enable must be a contiguous bool/uint8 [rows] tensor")
    a = _capi.TopkMixArgs()
    a.logits, a.embedding, a.out, a.row_enable = _ptr(logits), _ptr(embedding), _ptr(out), _ptr(row_enable)
    a.logits_row_stride = logits.stride(0) if rows > 1 else logits.shape[1]
    a.embedding_row_stride, a.out_row_stride = embedding.stride(0), (out.stride(0) if rows > 1 else H)
    a.rows, a.vocab, a.hidden, a.topk = rows, logits.shape[1], H, int(topk)
    _capi.check(lib, lib.tah_topk_mix(ctypes.byref(a), _stream(logits)), "tah_topk_mix")
    return out


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` of a fused gate|up projection, bf16 [rows, 2*I] -> [rows, I], in one launch."""
    lib = _lib.lib()
    _dev_check(gate_up)
    if gate_up.dim() != 2 or gate_up.dtype != torch.bfloat16 or gate_up.shape[1] % 16 or gate_up.stride(1) != 1:
        raise _capi.TahDuoError("silu_mul: gate_up must be bf16 [rows, 2*I] with I a multiple of 8 and a contiguous inner dimension")
    rows, inter = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((rows, inter), dtype=gate_up.dtype, device=gate_up.device)
    _capi.check(lib, lib.tah_silu_mul(_ptr(gate_up), _ptr(out), rows, inter, gate_up.stride(0) if rows > 1 else 2 * inter,
                                      inter, _stream(gate_up)), "tah_silu_mul")
    return out
