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


def add_score_drift(case, nats_per_key):
    """Makes every depth-0 score grow with the key index by about `nats_per_key` (on top of the random
    part): all queries get a common direction u added, key j gets j * t * u.  A running-maximum softmax
    then has to move its reference again and again (fast drift), or only every few tiles (slow drift)."""
    D = case["q1"].shape[-1]
    g = torch.Generator().manual_seed(1234)
    u = torch.randn(D, generator=g)
    u = u / u.norm()
    a = 4.0
    t = nats_per_key / (a * case["scale"])
    out = dict(case)
    out["q1"] = case["q1"] + a * u
    out["q2"] = case["q2"] + a * u
    k1 = case["k1"].clone()
    for b in range(len(case["cu_k1"]) - 1):
        lo, hi = int(case["cu_k1"][b]), int(case["cu_k1"][b + 1])
        j = torch.arange(hi - lo, dtype=k1.dtype)
        k1[lo:hi] += (j * t)[:, None, None] * u
    out["k1"] = k1
    return out


def make_masked_case(seed, B, Hq, Hkv, Tq, Tk, D=128, mask_dtype=torch.float32, per_head=False, p_hide=0.4):
    """Dense (B,H,T,D) bf16 q/k/v and an additive mask (B, 1|Hq, Tq, Tk): random small biases, a fraction
    p_hide of entries hidden with finfo.min (as tah_model.py:790) or -inf, every row keeping at least one
    visible key except row 0 of the last batch entry, which hides them all."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)
    q, k, v = rn(B, Hq, Tq, D), rn(B, Hkv, Tk, D), rn(B, Hkv, Tk, D)
    H = Hq if per_head else 1
    bias = (torch.randn(B, H, Tq, Tk, generator=g) * 0.5).to(mask_dtype).float()
    hide = torch.rand(B, H, Tq, Tk, generator=g) < p_hide
    hide[..., 0] = False
    hide[B - 1, :, 0, :] = True
    fm = torch.finfo(mask_dtype).min
    use_inf = torch.rand(B, H, Tq, Tk, generator=g) < 0.5
    mask = torch.where(hide, torch.where(use_inf, torch.tensor(float("-inf")), torch.tensor(fm)), bias).to(mask_dtype)
    return dict(q=q, k=k, v=v, mask=mask, scale=float(D) ** -0.5)


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


def make_decode_case(seed, lens, p_hard, Hq=16, Hkv=8, D=128, hard_new=None, std=1.0):
    """Decode-step inputs: packed depth-0 cache (every position, new token included), depth-1 cache
    (a Bernoulli(p_hard) subset of the positions, new token included when hard_new[b]), one depth-0
    query per sequence and one depth-1 query per hard sequence.  All float tensors bf16-representable."""
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: (torch.randn(*s, generator=g) * std).to(torch.bfloat16)
    lens = list(lens)
    nseq = len(lens)
    cu1 = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    k1, v1 = rn(int(cu1[-1]), Hkv, D), rn(int(cu1[-1]), Hkv, D)
    if hard_new is None:
        hard_new = (torch.rand(nseq, generator=g) < p_hard).tolist()
    pos2, cu2 = [], [0]
    for b, L in enumerate(lens):
        h = torch.rand(L, generator=g) < p_hard
        h[L - 1] = bool(hard_new[b])
        pos2 += torch.nonzero(h).flatten().tolist()
        cu2.append(len(pos2))
    k2, v2 = rn(len(pos2), Hkv, D), rn(len(pos2), Hkv, D)
    q1 = rn(nseq, Hq, D)
    hard_rows = [b for b in range(nseq) if hard_new[b]]
    q2 = rn(len(hard_rows), Hq, D)
    return dict(lens=lens, k1=k1, v1=v1, cu_k1=cu1, k2=k2, v2=v2, pos_k2=np.asarray(pos2, dtype=np.int32),
                cu_k2=np.asarray(cu2, dtype=np.int32), q1=q1, q2=q2, hard_rows=hard_rows,
                q_pos=np.asarray([L - 1 for L in lens], dtype=np.int32), scale=float(D) ** -0.5)


def build_slabs(c, capacity1, capacity2, device="cpu"):
    from tah_amd.kv_cache import KvSlabs
    hkv = c["k1"].shape[1]
    nseq = len(c["lens"])
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    s1 = KvSlabs(nseq, capacity1, hkv, with_pos=False, device=device)
    s2 = KvSlabs(nseq, capacity2, hkv, with_pos=True, device=device)
    s1.append(c["k1"].to(device), c["v1"].to(device), t(c["cu_k1"]))
    s2.append(c["k2"].to(device), c["v2"].to(device), t(c["cu_k2"]), pos_new=t(c["pos_k2"]))
    return s1, s2
