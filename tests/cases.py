"""Seeded synthetic inputs shared by the oracle tests, the GPU parity tests and the fixtures."""
from __future__ import annotations

import numpy as np
import torch


def make_varlen_case(seed, seqlens, p_hard, Hq=16, Hkv=8, D=128, dtype=torch.float32, std=1.0,
                     seqlens_k=None, extra_k2=0):
    """Packed varlen duo-causal inputs.

    seqlens: depth-0 query rows per sequence; seqlens_k (default = seqlens): depth-0
    key rows per sequence (>= seqlens; queries are bottom-right aligned).
    Hard rows are Bernoulli(p_hard) over query positions; depth-1 keys are the
    hard rows plus, when extra_k2 > 0, that many earlier cached depth-1 rows
    per sequence at positions below the first query position (if any exist).
    """
    g = torch.Generator().manual_seed(seed)
    seqlens = list(seqlens)
    seqlens_k = list(seqlens_k) if seqlens_k is not None else seqlens
    cu_q1 = np.concatenate([[0], np.cumsum(seqlens)]).astype(np.int32)
    cu_k1 = np.concatenate([[0], np.cumsum(seqlens_k)]).astype(np.int32)
    rn = lambda *s: (torch.randn(*s, generator=g) * std).to(dtype)
    T1q, T1k = int(cu_q1[-1]), int(cu_k1[-1])
    q1, k1, v1 = rn(T1q, Hq, D), rn(T1k, Hkv, D), rn(T1k, Hkv, D)
    pos_q2, pos_k2, cq2, ck2 = [], [], [0], [0]
    for lq, lk in zip(seqlens, seqlens_k):
        off = lk - lq
        hard = torch.rand(lq, generator=g) < p_hard
        hp = (torch.nonzero(hard).flatten() + off).tolist()
        pre = []
        if extra_k2 and off > 0:
            n = min(extra_k2, off)
            pre = sorted(torch.randperm(off, generator=g)[:n].tolist())
        pos_q2 += hp
        pos_k2 += pre + hp
        cq2.append(len(pos_q2))
        ck2.append(len(pos_k2))
    T2q, T2k = len(pos_q2), len(pos_k2)
    q2, k2, v2 = rn(T2q, Hq, D), rn(T2k, Hkv, D), rn(T2k, Hkv, D)
    return dict(
        q1=q1, k1=k1, v1=v1, cu_q1=cu_q1, cu_k1=cu_k1,
        q2=q2, k2=k2, v2=v2,
        pos_q2=np.asarray(pos_q2, dtype=np.int32), pos_k2=np.asarray(pos_k2, dtype=np.int32),
        cu_q2=np.asarray(cq2, dtype=np.int32), cu_k2=np.asarray(ck2, dtype=np.int32),
        scale=float(D) ** -0.5,
    )


VARLEN_KEYS = ("q1", "k1", "v1", "cu_q1", "cu_k1", "q2", "k2", "v2", "pos_q2", "pos_k2", "cu_q2", "cu_k2", "scale")


def varlen_args(case):
    return [case[k] for k in VARLEN_KEYS]


def make_dense_case(seed, B, T, p_hard, Hq=16, Hkv=8, D=128, dtype=torch.float32, left_pad=None):
    """Dense (B, T) batch as the reference's forward loop sees it."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g).to(dtype)
    q1, k1, v1 = rn(B, Hq, T, D), rn(B, Hkv, T, D), rn(B, Hkv, T, D)
    q2, k2, v2 = rn(B, Hq, T, D), rn(B, Hkv, T, D), rn(B, Hkv, T, D)
    valid = torch.ones(B, T, dtype=torch.long)
    if left_pad is not None:
        for b, n in enumerate(left_pad):
            valid[b, :n] = 0
    hard = (torch.rand(B, T, generator=g) < p_hard) & (valid == 1)
    return dict(q1=q1, k1=k1, v1=v1, q2=q2, k2=k2, v2=v2, hard=hard, valid=valid, scale=float(D) ** -0.5)


def dense_to_varlen(c):
    """Drop invalid tokens and pack a dense case into the varlen layout."""
    B, T = c["hard"].shape
    valid = c["valid"].bool()
    tok = lambda x: x.transpose(1, 2)  # (B,T,H,D)
    lens = valid.sum(1).tolist()
    cu1 = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    pos = (torch.cumsum(c["valid"], -1) - 1).clamp(min=0)
    sel2 = c["hard"] & valid
    cu2 = np.concatenate([[0], np.cumsum(sel2.sum(1).tolist())]).astype(np.int32)
    p2 = pos[sel2].numpy().astype(np.int32)
    return dict(
        q1=tok(c["q1"])[valid], k1=tok(c["k1"])[valid], v1=tok(c["v1"])[valid], cu_q1=cu1, cu_k1=cu1,
        q2=tok(c["q2"])[sel2], k2=tok(c["k2"])[sel2], v2=tok(c["v2"])[sel2],
        pos_q2=p2, pos_k2=p2, cu_q2=cu2, cu_k2=cu2, scale=c["scale"],
    )
