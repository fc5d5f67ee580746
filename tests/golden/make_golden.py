#!/usr/bin/env python3
"""Writes the golden fixtures of this directory from the CPU oracle.

The reference ships no tests or vectors for this path, and its arithmetic lives in un-vendored
third-party code, so these vectors come from this repository's own restatements: each expected
value below is produced by oracle/duo_ref.c (float64 accumulation, analytic backward) and is only
written after the independent float64 row-loop / torch-autograd restatement in
oracle/duo_oracle.py agrees with it.  Inputs are stored as bf16 bit patterns (uint16), expected
values as float32.  qk_prep_small.npz is the exception: its expected values are the outputs of the
third-party modules the reference calls (transformers' Qwen3RMSNorm / apply_rotary_pos_emb, installed
version recorded in the file), bf16 bit patterns.  Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import duo_oracle as O  # noqa: E402
from oracle import duo_ref as R  # noqa: E402
from tests.cases import make_decode_case, make_varlen_case, varlen_args  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def rounded(case):
    return {k: (v.to(torch.bfloat16).float() if torch.is_tensor(v) else v) for k, v in case.items()}


def prefill():
    c = rounded(make_varlen_case(4242, [21, 3, 40], 0.25, Hq=2, Hkv=1, D=128, seqlens_k=[21, 9, 40], extra_k2=2))
    g = torch.Generator().manual_seed(4243)
    do1 = torch.randn(c["q1"].shape, generator=g).to(torch.bfloat16).float()
    do2 = torch.randn(c["q2"].shape, generator=g).to(torch.bfloat16).float()
    o1, lse1, o2, lse2 = R.fwd(*varlen_args(c))
    a = O.duo_rows_f64(*varlen_args(c))
    for x, y in zip((o1, lse1, o2, lse2), a):
        np.testing.assert_allclose(x, y, atol=2e-6, rtol=1e-5)
    grads = R.bwd(*varlen_args(c), do1.numpy(), do2.numpy())
    t = {k: (v.double().requires_grad_(True) if torch.is_tensor(v) else v) for k, v in c.items()}
    r1, r2 = O.duo_varlen_torch(*varlen_args(t))
    ((r1 * do1.double()).sum() + (r2 * do2.double()).sum()).backward()
    for n, gc in zip(("q1", "k1", "v1", "q2", "k2", "v2"), grads):
        np.testing.assert_allclose(t[n].grad.numpy(), gc, atol=3e-6, rtol=1e-4)
    np.savez_compressed(
        os.path.join(HERE, "prefill_small.npz"),
        **{n: bits(c[n]) for n in ("q1", "k1", "v1", "q2", "k2", "v2")},
        **{n: c[n] for n in ("cu_q1", "cu_k1", "pos_q2", "pos_k2", "cu_q2", "cu_k2")},
        scale=np.float32(c["scale"]), do1=bits(do1), do2=bits(do2),
        o1=o1, lse1=lse1, o2=o2, lse2=lse2,
        **{"d" + n: gc for n, gc in zip(("q1", "k1", "v1", "q2", "k2", "v2"), grads)})


def decode():
    c = make_decode_case(4244, [70, 9, 130], 0.2, Hq=2, Hkv=1, hard_new=[True, False, True])
    f = lambda x: x.float().numpy()
    nseq = 3
    o0, l0 = O.duo_decode_f64(f(c["q1"]), f(c["k1"]), f(c["v1"]), c["cu_k1"], f(c["k2"]), f(c["v2"]), c["pos_k2"],
                              c["cu_k2"], c["q_pos"], [0] * nseq, c["scale"])
    hr = c["hard_rows"]
    q2 = np.zeros((nseq,) + tuple(c["q2"].shape[1:]))
    q2[hr] = f(c["q2"])
    o1, l1 = O.duo_decode_f64(q2, f(c["k1"]), f(c["v1"]), c["cu_k1"], f(c["k2"]), f(c["v2"]), c["pos_k2"], c["cu_k2"],
                              c["q_pos"], [1] * nseq, c["scale"])
    # second statement: the decode rows are the last rows of a varlen prefill with one query row per sequence
    cu_q1 = np.arange(nseq + 1, dtype=np.int32)
    cu_q2 = np.array([0, 1, 1, 2], dtype=np.int32)
    r = R.fwd(f(c["q1"]), f(c["k1"]), f(c["v1"]), cu_q1, c["cu_k1"], f(c["q2"]), f(c["k2"]), f(c["v2"]),
              c["q_pos"][hr], c["pos_k2"], cu_q2, c["cu_k2"], c["scale"])
    np.testing.assert_allclose(o0, r[0], atol=2e-6, rtol=1e-5)
    np.testing.assert_allclose(o1[hr], r[2], atol=2e-6, rtol=1e-5)
    np.savez_compressed(
        os.path.join(HERE, "decode_small.npz"),
        **{n: bits(c[n]) for n in ("q1", "k1", "v1", "q2", "k2", "v2")},
        cu_k1=c["cu_k1"], cu_k2=c["cu_k2"], pos_k2=c["pos_k2"], q_pos=c["q_pos"], hard_rows=np.asarray(hr, np.int32),
        lens=np.asarray(c["lens"], np.int32), scale=np.float32(c["scale"]),
        o_depth0=o0.astype(np.float32), lse_depth0=l0.astype(np.float32),
        o_depth1=o1[hr].astype(np.float32), lse_depth1=l1[hr].astype(np.float32))


def pack():
    g = torch.Generator().manual_seed(4245)
    mask = torch.rand(4, 50, generator=g) < 0.2
    mask[2] = False
    x = torch.randint(-1000, 1000, (4, 50, 3), generator=g)
    idx, cu = O.hard_index(mask)
    ridx, rcu = R.hard_index(mask.numpy())
    assert idx.tolist() == ridx.tolist() and cu.tolist() == rcu.tolist()
    assert idx.tolist() == mask.nonzero()[:, 1].tolist()
    pad, gx = O.gather_active(mask, x)
    assert torch.equal(gx[~pad], x[mask])
    amask = torch.rand(4, 50, generator=g) < 0.5
    dest = torch.full_like(x, -7)
    np.savez_compressed(
        os.path.join(HERE, "pack_small.npz"), mask=mask.numpy(), x=x.numpy(), idx=idx.numpy(), cu=cu.numpy(),
        pad_mask=pad.numpy(), gathered=gx.numpy(), assignment_mask=amask.numpy(),
        scattered=O.scatter_back(mask, gx, dest).numpy(),
        scattered_assigned=O.scatter_back(mask, gx, dest, assignment_mask=amask).numpy())


def qk_prep():
    """Expected values from the third-party modules themselves (the installed transformers'
    Qwen3RMSNorm and apply_rotary_pos_emb, bf16 on the CPU), written only if the oracle's restatement
    agrees with them to one bf16 unit in the last place on at most 0.1 % of the elements."""
    from transformers.models.qwen3 import modeling_qwen3 as m

    from oracle import qk_prep_ref as Q
    from tests.qk_prep_cases import make_case

    c = make_case(4246, 19, 4, 2, scale=1.5)
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16)
    qn, kn = m.Qwen3RMSNorm(128, eps=c["eps"]).to(torch.bfloat16), m.Qwen3RMSNorm(128, eps=c["eps"]).to(torch.bfloat16)
    with torch.no_grad():
        qn.weight.copy_(bf(c["qw"])), kn.weight.copy_(bf(c["kw"]))
        tq, tk = qn(bf(c["q"])).transpose(0, 1)[None], kn(bf(c["k"])).transpose(0, 1)[None]
        wq, wk = m.apply_rotary_pos_emb(tq, tk, bf(c["cos"])[None], bf(c["sin"])[None])
    wq, wk = wq[0].transpose(0, 1).contiguous(), wk[0].transpose(0, 1).contiguous()
    gq, gk = Q.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    for got, want in ((gq, wq.float().numpy()), (gk, wk.float().numpy())):
        ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64)) >> 16
        assert np.mean(got == want) > 0.999 and ulp.max() <= 1
    np.savez_compressed(
        os.path.join(HERE, "qk_prep_small.npz"),
        **{n: bits(bf(c[n])) for n in ("q", "k", "v", "qw", "kw", "cos", "sin")},
        pos=c["pos"], eps=np.float32(c["eps"]), q_out=bits(wq), k_out=bits(wk),
        transformers_version=np.array(__import__("transformers").__version__))


def topk_mix():
    """Top-k softmax mix (tah_model.py:57-75): distinct logits, so that torch's own topk / softmax / sum in bf16
    (the reference's call sequence, library routines) and the oracle name the same rows; the fixture keeps the
    oracle's output after the two agree to one bf16 step."""
    from oracle.topk_mix_ref import topk_mix as ref
    from tests.topk_mix_cases import make_case

    logits, emb = make_case(4247, 3, 1200, 48, distinct=True)
    k = 100
    out = ref(logits, emb, k)
    lg, em = torch.from_numpy(logits).to(torch.bfloat16), torch.from_numpy(emb).to(torch.bfloat16)
    tv, ti = torch.topk(lg, k=k, dim=-1)
    lib = torch.sum(torch.softmax(tv, -1).unsqueeze(-1) * em[ti], dim=-2).to(em.dtype).float().numpy()
    assert (np.abs(out - lib) <= np.maximum(np.abs(lib), 1e-3) * 2.0 ** -7).all() and (out == lib).mean() > 0.9
    np.savez_compressed(os.path.join(HERE, "topk_mix_small.npz"), logits=logits, emb=emb, k=np.int32(k), out=out)


if __name__ == "__main__":
    prefill()
    decode()
    pack()
    qk_prep()
    topk_mix()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
