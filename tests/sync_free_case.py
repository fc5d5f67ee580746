"""The forward loop around one attention layer (tah_model.py:580-623) at both depths with every host
synchronisation of the pack removed: ``tah_amd.pack.HOST_SYNC = False``, ``gather_active(max_active=...)``.
On the GPU the loop runs under ``torch.cuda.set_sync_debug_mode("error")``, which turns any ``.item()`` /
``.cpu()`` / ``nonzero`` on a device tensor into an exception.  Shared by the CPU-shim and the GPU test."""
import types

import numpy as np
import torch

from oracle import duo_oracle as O
from tests.cases import make_dense_case


def run(device, *, B=3, T=60, p=0.25, left_pad=(0, 11, 30), seed=70, Hq=4, Hkv=2, with_decode=True):
    from tah_amd import pack
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.cache import TaHDuoCache

    layer = types.SimpleNamespace(layer_idx=0, num_key_value_groups=Hq // Hkv)
    c = make_dense_case(seed, B=B, T=T + 1, p_hard=p, Hq=Hq, Hkv=Hkv, D=128, left_pad=list(left_pad))
    c["hard"][:, T] = torch.tensor([True] + [False] * (B - 1))  # the decode step: one hard row, the rest pad rows
    bf = lambda x: x.to(torch.bfloat16).to(device)
    tok = lambda x: x.transpose(1, 2)
    valid_all, hard_all = c["valid"].to(device), c["hard"].to(device)
    pos_all = (torch.cumsum(valid_all, -1) - 1).clamp(min=0)
    W = int(c["hard"][:, :T].sum(1).max()) + 2  # a bound the caller knows (e.g. a fixed budget of hard tokens)
    t = {k: bf(c[k]) for k in ("q1", "k1", "v1", "q2", "k2", "v2")}
    cache = TaHDuoCache().enable_slabs(T + 4, T + 4) if with_decode else TaHDuoCache()

    def loop(sl, width):
        pos, valid, hard = pos_all[:, sl], valid_all[:, sl], hard_all[:, sl]
        m0 = build_attention_mask(pos, valid, cache, 0)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
        k, v = cache.update(t["k1"][:, :, sl], t["v1"][:, :, sl], 0)
        o1, _ = duo_attention_forward(layer, t["q1"][:, :, sl], k, v, m0, scaling=c["scale"])
        pad, q2, k2, v2, pos2, val2 = pack.gather_active(hard, tok(t["q2"][:, :, sl]), tok(t["k2"][:, :, sl]),
                                                         tok(t["v2"][:, :, sl]), pos, valid, max_active=width)
        m1 = build_attention_mask(pos2, val2, cache, 1)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 1, pos2, val2
        k, v = cache.update(tok(k2), tok(v2), 0)
        o2, _ = duo_attention_forward(layer, tok(q2), k, v, m1, scaling=c["scale"])
        back = pack.scatter_back(hard, o2, torch.zeros_like(o1))
        return o1, o2, pad, back

    old = pack.HOST_SYNC
    pack.HOST_SYNC = False
    if device != "cpu":
        torch.cuda.synchronize()
        torch.cuda.set_sync_debug_mode("error")
    try:
        with torch.no_grad():
            o1, o2, pad, back = loop(slice(0, T), W)
            d1, d2, dpad, dback = loop(slice(T, T + 1), 1) if with_decode else (None,) * 4
    finally:
        if device != "cpu":
            torch.cuda.set_sync_debug_mode("default")
        pack.HOST_SYNC = old
    assert int(pad.overflow) == 0

    # the reference formulation on the host
    r = lambda x: x.to(torch.bfloat16).float()
    sl = slice(0, T)
    w1, w2, wpad = O.duo_prefill_dense(r(c["q1"][:, :, sl]), r(c["k1"][:, :, sl]), r(c["v1"][:, :, sl]), r(c["q2"][:, :, sl]),
                                       r(c["k2"][:, :, sl]), r(c["v2"][:, :, sl]), c["hard"][:, sl], c["scale"],
                                       valid_mask=c["valid"][:, sl])
    valid = c["valid"][:, sl].bool()
    np.testing.assert_allclose(o1.cpu()[valid].float().numpy(), w1[valid].numpy(), atol=2e-2, rtol=2e-2)
    assert (o1.cpu()[~valid] == 0).all()
    n2 = wpad.shape[1]
    assert pad.shape[1] == W and torch.equal(pad.cpu()[:, :n2], wpad) and pad.cpu()[:, n2:].all()
    np.testing.assert_allclose(o2.cpu()[:, :n2][~wpad].float().numpy(), w2[~wpad].numpy(), atol=2e-2, rtol=2e-2)
    assert (o2.cpu()[pad.cpu()] == 0).all()
    hard0 = c["hard"][:, sl] & valid
    assert torch.equal(back.cpu()[hard0], o2.cpu()[~pad.cpu()]) and (back.cpu()[~hard0] == 0).all()
    if with_decode:
        # the decode step against the dense formulation over the whole (T+1)-token batch: last position
        f1, f2, fpad = O.duo_prefill_dense(*(r(c[n]) for n in ("q1", "k1", "v1", "q2", "k2", "v2")), c["hard"], c["scale"],
                                           valid_mask=c["valid"])
        np.testing.assert_allclose(d1.cpu()[:, 0].float().numpy(), f1[:, T].numpy(), atol=2e-2, rtol=2e-2)
        # row 0 is the hard one: its depth-1 output is the last packed entry of row 0
        last0 = int((c["hard"][0] & c["valid"][0].bool()).sum()) - 1
        np.testing.assert_allclose(d2.cpu()[0, 0].float().numpy(), f2[0, last0].numpy(), atol=2e-2, rtol=2e-2)
        assert (d2.cpu()[1:] == 0).all() and dpad.cpu()[:, 0].tolist() == [False] + [True] * (B - 1)
        assert cache.slabs(0, 0).len.tolist() == c["valid"].sum(1).tolist()
        assert cache.slabs(0, 1).len.tolist() == (c["hard"] & c["valid"].bool()).sum(1).tolist()
    return True
