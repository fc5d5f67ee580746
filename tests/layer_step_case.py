"""One attention layer's decode loop composed from the library's pieces -- fused q/k preparation with
KV append into slabs, then the split-K decode kernel -- against a plain restatement: the oracle's
RMSNorm + rotary on every row, growing per-sequence lists of K and V, float64 softmax over the rows a
query may see (depth-0 rows up to its position; at depth 1 also the depth-1 rows up to its position)."""
import numpy as np
import torch

from oracle import qk_prep_ref as R


def run(device, qk_norm_rope, KvSlabs, decode, *, B=3, hq=4, hkv=2, prompt=(37, 5, 64), steps=3, seed=0, cap=96):
    g = np.random.default_rng(seed)
    D, eps, scale, grp = 128, 1e-6, 128 ** -0.5, hq // hkv
    rb = lambda *s: R.bf16_round(g.standard_normal(s).astype(np.float32))
    qw, kw = R.bf16_round((1 + 0.1 * g.standard_normal(D)).astype(np.float32)), R.bf16_round((1 + 0.1 * g.standard_normal(D)).astype(np.float32))
    T = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).to(device)
    I = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    s0, s1 = KvSlabs(B, cap, hkv, with_pos=False, device=device), KvSlabs(B, cap, hkv, with_pos=True, device=device)
    ref0 = [([], []) for _ in range(B)]           # per sequence: depth-0 K rows, V rows
    ref1 = [([], [], []) for _ in range(B)]       # depth-1 K rows, V rows, positions
    worst = 0.0

    def prep_ref(q, k, pos):
        cos, sin = R.rotary_tables(np.asarray(pos))
        return R.qk_prep(q, k, qw, kw, cos, sin, eps), (cos, sin)

    def attend(qrow, keys, vals):  # qrow [hq, D]; keys/vals lists of [hkv, D]
        K, V = np.stack(keys).astype(np.float64), np.stack(vals).astype(np.float64)
        out = np.zeros((hq, D))
        for h in range(hq):
            s = K[:, h // grp] @ qrow[h].astype(np.float64) * scale
            p = np.exp(s - s.max())
            out[h] = (p / p.sum()) @ V[:, h // grp]
        return out

    # prompt: every row through the preparation kernel, K and V appended (depth 0 only)
    rows = sum(prompt)
    cu = np.concatenate([[0], np.cumsum(prompt)]).astype(np.int32)
    pos = np.concatenate([np.arange(n) for n in prompt])
    q, k, v = rb(rows, hq, D), rb(rows, hkv, D), rb(rows, hkv, D)
    (_, kr), (cos, sin) = prep_ref(q, k, pos)
    qk_norm_rope(T(q), T(k), T(qw), T(kw), T(cos), T(sin), eps, v=T(v), cache=s0, cu_new=I(cu))
    for b in range(B):
        for r in range(cu[b], cu[b + 1]):
            ref0[b][0].append(kr[r]), ref0[b][1].append(v[r])
    lens = list(prompt)
    for step in range(steps):
        hard = [(b + step) % 2 == 0 for b in range(B)]
        # depth 0: one new token per sequence
        q, k, v = rb(B, hq, D), rb(B, hkv, D), rb(B, hkv, D)
        (qr, kr), (cos, sin) = prep_ref(q, k, lens)
        q_dev, _ = qk_norm_rope(T(q), T(k), T(qw), T(kw), T(cos), T(sin), eps, v=T(v), cache=s0, cu_new=I(np.arange(B + 1)))
        o = decode(q_dev, I(np.arange(B)), I(lens), s0, None, scale=scale, depth=0)
        for b in range(B):
            ref0[b][0].append(kr[b]), ref0[b][1].append(v[b])
            want = attend(qr[b], ref0[b][0], ref0[b][1])
            worst = max(worst, float(np.abs(o[b].float().cpu().numpy() - want).max()))
        # depth 1: the hard sequences run the token again, same position, seeing both caches
        hs = [b for b in range(B) if hard[b]]
        if hs:
            n = len(hs)
            q, k, v = rb(n, hq, D), rb(n, hkv, D), rb(n, hkv, D)
            hpos = [lens[b] for b in hs]
            (qr, kr), (cos, sin) = prep_ref(q, k, hpos)
            q_dev, _ = qk_norm_rope(T(q), T(k), T(qw), T(kw), T(cos), T(sin), eps, v=T(v), cache=s1, cu_new=I(np.arange(n + 1)),
                                    pos_new=I(hpos), slot_of=I(hs))
            o = decode(q_dev, I(hs), I(hpos), s0, s1, scale=scale, depth=1)
            for i, b in enumerate(hs):
                ref1[b][0].append(kr[i]), ref1[b][1].append(v[i]), ref1[b][2].append(lens[b])
                want = attend(qr[i], ref0[b][0] + ref1[b][0], ref0[b][1] + ref1[b][1])
                worst = max(worst, float(np.abs(o[i].float().cpu().numpy() - want).max()))
        lens = [n + 1 for n in lens]
    assert s0.len.cpu().tolist() == lens and int(s0.overflow) == 0 and int(s1.overflow) == 0
    return worst
