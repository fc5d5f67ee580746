"""Host layer (pack API, cache protocol, mask carrier, HF attention callable) driven the way the reference's
forward loop drives it, with the kernels running on the CPU execution shim.  No GPU."""
import types

import numpy as np
import pytest
import torch

from oracle import duo_oracle as O
from tests import emu_util
from tests.cases import make_dense_case

pytestmark = pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")


@pytest.fixture()
def emu():
    with emu_util.emulated() as lib:
        yield lib


@pytest.mark.parametrize("seed,p", [(0, 0.3), (1, 0.0), (2, 1.0)])
def test_gather_scatter_match_reference_semantics(emu, seed, p):
    from tah_amd.pack import gather_active, scatter_back
    g = torch.Generator().manual_seed(seed)
    B, S = 3, 21
    mask = torch.rand(B, S, generator=g) < p
    if seed == 0:
        mask[1] = False
    x = torch.randn(B, S, 8, generator=g).to(torch.bfloat16)
    ids = torch.arange(B * S).view(B, S)
    got = gather_active(mask, x, ids, None)
    want = O.gather_active(mask, x, ids, None)
    assert got[3] is None and len(got) == 4
    for a, b in zip(got[:3], want[:3]):
        assert a.shape == b.shape and a.dtype == b.dtype and torch.equal(a, b)
    lab = gather_active(mask, ids, pad_value=-100)[1]
    assert torch.equal(lab, O.gather_active(mask, ids, pad_value=-100)[1])
    dest = torch.full((B, S, 8), -7.0).to(torch.bfloat16)
    assert torch.equal(scatter_back(mask, got[1], dest), O.scatter_back(mask, want[1], dest))
    amask = torch.rand(B, S, generator=g) < 0.5
    assert torch.equal(scatter_back(mask, got[1], dest, assignment_mask=amask),
                       O.scatter_back(mask, want[1], dest, assignment_mask=amask))
    d2 = dest.clone()
    assert scatter_back(mask, got[1], d2, in_place=True) is d2 and torch.equal(d2, O.scatter_back(mask, want[1], dest))
    fin = torch.zeros(B, S, dtype=torch.bool)
    fm = torch.ones_like(got[0])
    scatter_back(mask, fm, fin, in_place=True)
    assert torch.equal(fin, mask)


def test_gather_scatter_autograd(emu):
    from tah_amd.pack import gather_active, scatter_back
    g = torch.Generator().manual_seed(5)
    B, S = 2, 9
    mask = torch.rand(B, S, generator=g) < 0.5
    x = torch.randn(B, S, 4, generator=g, requires_grad=True)
    xr = x.detach().clone().requires_grad_(True)
    w = torch.randn(B, int(mask.sum(1).max()), 4, generator=g)
    (gather_active(mask, x)[1] * w).sum().backward()
    pad, gx = O.gather_active(mask, xr)
    idx = torch.nonzero(mask)
    ref = torch.zeros_like(xr)
    for b in range(B):
        cols = torch.nonzero(mask[b]).flatten()
        ref[b, cols] = w[b, : len(cols)]
    assert torch.equal(x.grad, ref)
    src = torch.randn(B, w.shape[1], 4, generator=g, requires_grad=True)
    dest = torch.randn(B, S, 4, generator=g, requires_grad=True)
    amask = torch.rand(B, S, generator=g) < 0.6
    wo = torch.randn(B, S, 4, generator=g)
    out = scatter_back(mask, src, dest, assignment_mask=amask)
    assert torch.equal(out.detach(), O.scatter_back(mask, src.detach(), dest.detach(), assignment_mask=amask))
    (out * wo).sum().backward()
    fm = mask & amask
    assert torch.equal(dest.grad, torch.where(fm[..., None], torch.zeros_like(wo), wo))
    gs = torch.zeros_like(src)
    for b in range(B):
        for k, c in enumerate(torch.nonzero(mask[b]).flatten().tolist()):
            if fm[b, c]:
                gs[b, k] = wo[b, c]
    assert torch.equal(src.grad, gs)


def _layer(layer_idx=0):
    return types.SimpleNamespace(layer_idx=layer_idx, num_key_value_groups=2)


def _forward_two_depths(c, cache, requires_grad=False, device="cpu"):
    """The reference's forward loop around one attention layer (tah_model.py:580-623), two depths."""
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.pack import gather_active
    bf = lambda x: x.to(torch.bfloat16).to(device)
    c = dict(c, hard=c["hard"].to(device), valid=c["valid"].to(device))
    B, T = c["hard"].shape
    valid = c["valid"]
    pos = (torch.cumsum(valid, -1) - 1).clamp(min=0)
    t = {k: bf(c[k]).clone().requires_grad_(requires_grad) for k in ("q1", "k1", "v1", "q2", "k2", "v2")}
    m0 = build_attention_mask(pos, valid, cache, 0, dtype=torch.bfloat16)
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
    k, v = cache.update(t["k1"], t["v1"], 0)
    o1, none = duo_attention_forward(_layer(), t["q1"], k, v, m0, dropout=0.0, scaling=c["scale"])
    assert none is None and o1.shape == (B, T, t["q1"].shape[1], 128)
    tok = lambda x: x.transpose(1, 2)
    pad, q2, k2, v2, pos2, val2 = gather_active(c["hard"], tok(t["q2"]), tok(t["k2"]), tok(t["v2"]), pos, valid)
    if pad.shape[1] == 0:
        return t, o1, None, pad
    m1 = build_attention_mask(pos2, val2, cache, 1, dtype=torch.bfloat16)
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 1, pos2, val2
    k, v = cache.update(tok(k2), tok(v2), 0)
    o2, _ = duo_attention_forward(_layer(), tok(q2), k, v, m1, scaling=c["scale"])
    return t, o1, o2, pad


def _forward_two_depths_reference_style(c, cache, device="cpu"):
    """The same loop as the reference runs it today: a dense additive mask in the mask slot and the
    concatenated cache as key/value (tah_model.py:604-623, causal_cache.py:97).  Exercises the
    additive-mask compatibility mode of the attention callable."""
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.pack import gather_active
    bf = lambda x: x.to(torch.bfloat16).to(device)
    c = dict(c, hard=c["hard"].to(device), valid=c["valid"].to(device))
    valid = c["valid"]
    pos = (torch.cumsum(valid, -1) - 1).clamp(min=0)
    t = {k: bf(c[k]) for k in ("q1", "k1", "v1", "q2", "k2", "v2")}
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
    dense0 = build_attention_mask(pos, valid, cache, 0, dtype=torch.bfloat16).dense(torch.bfloat16)
    cache.update(t["k1"], t["v1"], 0)
    K, V = cache.get_cache_upto_iter(0, 0)
    o1, _ = duo_attention_forward(_layer(), t["q1"], K, V, dense0, dropout=0.0, scaling=c["scale"])
    tok = lambda x: x.transpose(1, 2)
    pad, q2, k2, v2, pos2, val2 = gather_active(c["hard"], tok(t["q2"]), tok(t["k2"]), tok(t["v2"]), pos, valid)
    if pad.shape[1] == 0:
        return o1, None, pad
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 1, pos2, val2
    dense1 = build_attention_mask(pos2, val2, cache, 1, dtype=torch.bfloat16).dense(torch.bfloat16)
    cache.update(tok(k2), tok(v2), 0)
    K, V = cache.get_cache_upto_iter(0, 1)
    o2, _ = duo_attention_forward(_layer(), tok(q2), K, V, dense1, scaling=c["scale"])
    return o1, o2, pad


def _oracle_two_depths(c):
    r = lambda x: x.to(torch.bfloat16).float()
    return O.duo_prefill_dense(r(c["q1"]), r(c["k1"]), r(c["v1"]), r(c["q2"]), r(c["k2"]), r(c["v2"]), c["hard"],
                               c["scale"], valid_mask=c["valid"])


def test_forward_loop_with_launch_order_table(emu, monkeypatch):
    """With the launch-order table switched on for every call size the loop returns what it returns without
    it; one table is built per depth and the backward pass runs with it."""
    from tah_amd import attention, ops
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(33, B=3, T=40, p_hard=0.25, Hq=2, Hkv=1, D=128, left_pad=[0, 6, 22])
    _, w1, w2, _ = _forward_two_depths(c, TaHDuoCache())
    built = []
    real = ops.duo_schedule
    monkeypatch.setattr(ops, "duo_schedule", lambda *a: built.append(1) or real(*a))
    monkeypatch.setattr(attention, "SCHEDULE_MIN_ROW_HEADS", 0)
    monkeypatch.setattr(attention, "SCHEDULE_MIN_MEAN_ROWS", 0)
    cache = TaHDuoCache()
    t, o1, o2, _ = _forward_two_depths(c, cache, requires_grad=True)
    assert len(built) == 2 and torch.equal(o1, w1) and torch.equal(o2, w2)
    (o1.float().sum() + o2.float().sum()).backward()
    assert all(t[k].grad is not None for k in ("q1", "k1", "v1"))


@pytest.mark.parametrize("left_pad,no_sync_rows", [(None, 4096), ([0, 9], 4096), ([0, 9], 0)])
def test_forward_loop_matches_dense_reference(emu, monkeypatch, left_pad, no_sync_rows):
    """(no_sync_rows = 0: every block reads its valid count back and packs to it, as large blocks do.)"""
    import tah_amd.attention as A
    from tah_amd.cache import TaHDuoCache
    monkeypatch.setattr(A, "NO_SYNC_ROWS", no_sync_rows)
    c = make_dense_case(31, B=2, T=40, p_hard=0.25, Hq=4, Hkv=2, D=128, left_pad=left_pad)
    cache = TaHDuoCache()
    _, o1, o2, pad = _forward_two_depths(c, cache)
    w1, w2, wpad = _oracle_two_depths(c)
    assert torch.equal(pad, wpad)
    valid = c["valid"].bool()
    np.testing.assert_allclose(o1[valid].float().numpy(), w1[valid].numpy(), atol=2e-2, rtol=2e-2)
    assert (o1[~valid] == 0).all()
    np.testing.assert_allclose(o2[~pad].float().numpy(), w2[~pad].numpy(), atol=2e-2, rtol=2e-2)
    assert (o2[pad] == 0).all()
    # cache protocol: same lengths / metadata as the reference's cache after the same writes
    n2 = pad.shape[1]
    assert cache.get_seq_length(0) == 40 and cache.get_cache_length(0) == 40 + n2
    assert cache.get_kv_length_upto_iter(0, 1) == 40 + n2 and cache.get_cache_length(0, 1) == n2
    assert cache.get_cache_iter_index_upto_iter(0, 1).tolist() == [0] * 40 + [1] * n2
    assert cache.get_position_id_upto_iter(0, 1).shape == (2, 40 + n2)
    assert cache.get_valid_mask_upto_iter(0, 0).tolist() == c["valid"].tolist()
    assert cache.has_layer(0) and not cache.has_layer(1) and cache.batch_size == 2
    K, V = cache.get_cache_upto_iter(0, 1)
    assert K.shape == (2, 2, 40 + n2, 128)
    with pytest.raises(AssertionError):
        cache.update(K[:1], V[:1], 0)


def test_reference_style_loop_with_dense_masks_matches_dense_reference(emu):
    """Compatibility mode end to end: dense masks + concatenated cache, as the reference calls SDPA today."""
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(33, B=2, T=40, p_hard=0.25, Hq=4, Hkv=2, D=128, left_pad=[0, 9])
    o1, o2, pad = _forward_two_depths_reference_style(c, TaHDuoCache())
    w1, w2, wpad = _oracle_two_depths(c)
    valid = c["valid"].bool()
    np.testing.assert_allclose(o1[valid].float().numpy(), w1[valid].numpy(), atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(o2[~pad].float().numpy(), w2[~pad].numpy(), atol=2e-2, rtol=2e-2)


def test_dense_mask_of_carrier_equals_reference_mask(emu):
    from tah_amd.attention import build_attention_mask
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(32, B=2, T=12, p_hard=0.4, Hq=2, Hkv=1, D=128, left_pad=[3, 0])
    cache, ocache = TaHDuoCache(), O.OracleCache()
    pos = (torch.cumsum(c["valid"], -1) - 1).clamp(min=0)
    m = build_attention_mask(pos, c["valid"], cache, 0, torch.float32)
    assert torch.equal(m.dense(), O.build_attention_mask(pos, c["valid"], ocache, 0, torch.float32))
    for ch in (cache, ocache):
        ch.current_iter_depth, ch.position_ids_to_cache, ch.valid_mask_to_cache = 0, pos, c["valid"]
        ch.update(c["k1"].to(torch.bfloat16), c["v1"].to(torch.bfloat16), 0)
    pad, pos2, val2 = O.gather_active(c["hard"], pos, c["valid"])
    m1 = build_attention_mask(pos2, val2, cache, 1, torch.float32)
    assert torch.equal(m1.dense(), O.build_attention_mask(pos2, val2, ocache, 1, torch.float32))
    assert build_attention_mask(pos[:, :0], c["valid"][:, :0], None, 0) is None


def test_forward_loop_gradients(emu):
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(33, B=1, T=36, p_hard=0.3, Hq=2, Hkv=1, D=128)
    t, o1, o2, pad = _forward_two_depths(c, TaHDuoCache(), requires_grad=True)
    g = torch.Generator().manual_seed(1)
    w1, w2 = torch.randn(o1.shape, generator=g), torch.randn(o2.shape, generator=g)
    ((o1.float() * w1).sum() + (o2.float() * w2).sum()).backward()
    ref = {k: c[k].to(torch.bfloat16).double().requires_grad_(True) for k in t}
    r1, r2, rpad = O.duo_prefill_dense(ref["q1"], ref["k1"], ref["v1"], ref["q2"], ref["k2"], ref["v2"], c["hard"], c["scale"])
    ((r1 * w1.to(torch.bfloat16).double()).sum() + (r2 * w2.to(torch.bfloat16).double()).sum()).backward()
    hard = c["hard"][0]
    for n in ("q1", "k1", "v1", "q2", "k2", "v2"):
        a, b = t[n].grad.float(), ref[n].grad.float()
        if n.endswith("2"):  # only hard rows of the depth-1 projections take part
            assert (a[0, :, ~hard] == 0).all()
        err = (a - b).abs().max() / b.abs().max()
        assert err < 3e-2, (n, float(err))


def test_decode_steps_through_cache_and_callable(emu):
    """Prefill then decode steps at both depths with slabs; compare with the dense reference over the grown cache."""
    from tests.decode_steps_case import run
    cache, n1 = run("cpu", steps=4, force_hard=[[0], [], [0, 1], [1]])
    assert n1 == 3  # three of the four decode steps had a depth-1 pass (one with a pad row, one with both rows hard)
    # decode steps leave K/V in the slabs only: the concatenating getter says so instead of returning a partial cache
    from tah_amd import TahDuoError
    with pytest.raises(TahDuoError):
        cache.get_cache_upto_iter(0, 0)


def test_slab_overflow_raises_through_cache_update(emu):
    """A generation that outgrows the slab capacity fails on the host at the write, not silently on the device."""
    from tah_amd import TahDuoError
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(35, B=1, T=9, p_hard=0.0, Hq=2, Hkv=1, D=128)
    bf = lambda x: x.to(torch.bfloat16)
    cache = TaHDuoCache().enable_slabs(6, 4)
    pos_all = torch.arange(9)[None]
    one = torch.ones(1, 9, dtype=torch.long)

    def feed(lo, hi):
        sl = slice(lo, hi)
        m = build_attention_mask(pos_all[:, sl], one[:, sl], cache, 0)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos_all[:, sl], one[:, sl]
        k, v = cache.update(bf(c["k1"][:, :, sl]), bf(c["v1"][:, :, sl]), 0)
        return duo_attention_forward(_layer(), bf(c["q1"][:, :, sl]), k, v, m, scaling=c["scale"])[0]

    with torch.no_grad():
        feed(0, 5)
        feed(5, 6)
        with pytest.raises(TahDuoError, match="capacity"):
            feed(6, 7)
    assert int(cache.slabs(0, 0).overflow) == 0 and cache.slabs(0, 0).len.tolist() == [6]


def _loops_over_depths(c, deeper, requires_grad=False, device="cpu", position_ids=None):
    """The reference's forward loop (tah_model.py:580-623) over more than two latent iterations, run twice on the same
    bf16 inputs: through this package (TaHDuoCache, DuoMask, duo_attention_forward) and through the dense restatement
    (list cache, dense mask, softmax in float64).  ``deeper``: [(active mask (B, T), q, k, v dense (B, H, T, D)), ...]
    for depths 2, 3, ...; depth 1 uses c["hard"] and q2 / k2 / v2.  Returns per depth (ours, reference, pad mask), and
    the leaves of both runs."""
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.cache import TaHDuoCache
    from tah_amd.pack import gather_active
    cache, ocache = TaHDuoCache(), O.OracleCache()
    valid = c["valid"]
    pos = (torch.cumsum(valid, -1) - 1).clamp(min=0) if position_ids is None else position_ids
    levels = [(None, c["q1"], c["k1"], c["v1"]), (c["hard"], c["q2"], c["k2"], c["v2"])] + list(deeper)
    tok = lambda x: x.transpose(1, 2)
    leaves, rleaves, outs = [], [], []
    for depth, (active, q, k, v) in enumerate(levels):
        t = [x.to(torch.bfloat16).to(device).requires_grad_(requires_grad) for x in (q, k, v)]
        r = [x.to(torch.bfloat16).double().requires_grad_(requires_grad) for x in (q, k, v)]
        leaves.append(t)
        rleaves.append(r)
        if active is None:
            (tq, tk, tv), (rq, rk, rv), p, vl, rp, rvl, pad = t, r, pos.to(device), valid.to(device), pos, valid, None
        else:
            pad, tq, tk, tv, p, vl = gather_active(active.to(device), tok(t[0]), tok(t[1]), tok(t[2]), pos.to(device), valid.to(device))
            rpad, rq, rk, rv, rp, rvl = O.gather_active(active, tok(r[0]), tok(r[1]), tok(r[2]), pos, valid)
            pad = pad.cpu()
            assert torch.equal(pad, rpad) and torch.equal(p.cpu(), rp) and torch.equal(vl.cpu(), rvl)
            tq, tk, tv, rq, rk, rv = (tok(x) for x in (tq, tk, tv, rq, rk, rv))
        m = build_attention_mask(p, vl, cache, depth, dtype=torch.bfloat16)
        om = O.build_attention_mask(rp, rvl, ocache, depth, torch.float64)
        assert torch.equal(m.dense(torch.float64).cpu(), om)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = depth, p, vl
        ocache.current_iter_depth, ocache.position_ids_to_cache, ocache.valid_mask_to_cache = depth, rp, rvl
        kk, vv = cache.update(tk, tv, 0)
        o, _ = duo_attention_forward(_layer(), tq, kk, vv, m, scaling=c["scale"])
        K, V = ocache.update(rk, rv, 0)
        outs.append((o, O.sdpa_dense(rq, K, V, om, c["scale"]), pad))
    assert cache.get_cache_iter_index_upto_iter(0, len(levels) - 1).tolist() == ocache.get_cache_iter_index_upto_iter(0, len(levels) - 1).tolist()
    return outs, leaves, rleaves


def _deeper_levels(c, seed, n):
    """n more latent iterations over shrinking subsets of the hard tokens, with projections of their own."""
    g = torch.Generator().manual_seed(seed)
    B, Hq, T, D = c["q1"].shape
    Hkv = c["k1"].shape[1]
    active, out = c["hard"], []
    for _ in range(n):
        active = active & (torch.rand(B, T, generator=g) < 0.6)
        out.append((active, torch.randn(B, Hq, T, D, generator=g), torch.randn(B, Hkv, T, D, generator=g),
                    torch.randn(B, Hkv, T, D, generator=g)))
    return out


@pytest.mark.parametrize("left_pad,n_deeper", [(None, 1), ([0, 7], 2)])
def test_forward_loop_over_three_and_four_depths_matches_dense_reference(emu, left_pad, n_deeper):
    """The reference's mask and cache take any depth (tah_model.py:788, causal_cache.py:101-158; both deciders default
    to max_iter = 3): a query at depth d sees the keys of depths 0..d at or before its position."""
    c = make_dense_case(41, B=2, T=44, p_hard=0.5, Hq=4, Hkv=2, D=128, left_pad=left_pad)
    deeper = _deeper_levels(c, 42, n_deeper)
    assert all(int(lv[0].sum()) > 0 for lv in deeper)
    check_depth_outputs(c, _loops_over_depths(c, deeper)[0])


def check_depth_outputs(c, outs):
    valid = c["valid"].bool()
    for depth, (o, w, pad) in enumerate(outs):
        o, w = o.detach().cpu(), w.detach()
        keep = valid if pad is None else ~pad
        np.testing.assert_allclose(o[keep].float().numpy(), w[keep].float().numpy(), atol=2e-2, rtol=2e-2, err_msg=f"depth {depth}")
        assert (o[~keep] == 0).all()


def test_forward_loop_over_three_depths_gradients(emu):
    c = make_dense_case(43, B=2, T=30, p_hard=0.5, Hq=2, Hkv=1, D=128, left_pad=[0, 5])
    deeper = _deeper_levels(c, 44, 1)
    check_depth_gradients(c, *_loops_over_depths(c, deeper, requires_grad=True))


def check_depth_gradients(c, outs, leaves, rleaves):
    g = torch.Generator().manual_seed(2)
    loss = rloss = 0.0
    for o, w, pad in outs:
        wt = torch.randn(o.shape, generator=g).to(torch.bfloat16)
        if pad is not None:
            wt = torch.where(pad[..., None, None], torch.zeros_like(wt), wt)   # (pad rows: zeros here, anything there)
        else:
            wt = torch.where(c["valid"].bool()[..., None, None], wt, torch.zeros_like(wt))
        loss = loss + (o.float() * wt.float().to(o.device)).sum()
        rloss = rloss + (w * wt.double()).sum()
    loss.backward()
    rloss.backward()
    for depth, (t, r) in enumerate(zip(leaves, rleaves)):
        for name, a, b in zip("qkv", t, r):
            err = (a.grad.float().cpu() - b.grad.float()).abs().max() / b.grad.abs().max().clamp_min(1e-6).float()
            assert err < 3e-2, (depth, name, float(err))


def caller_position_ids(c, seed, kind):
    """Position ids that are not the tokens' ranks: ``documents``: several documents packed into one row, positions
    starting again at 0 in each; ``shuffled``: a random permutation of the ranks with an offset; ``coarse``: many
    tokens sharing a position."""
    g = torch.Generator().manual_seed(seed)
    B, T = c["valid"].shape
    rank = (torch.cumsum(c["valid"], -1) - 1).clamp(min=0)
    if kind == "documents":
        starts = torch.rand(B, T, generator=g) < 0.08
        starts[:, 0] = True
        doc_start = torch.cummax(torch.where(starts, rank, torch.zeros_like(rank)), dim=-1).values
        return rank - doc_start
    if kind == "shuffled":
        return torch.stack([torch.randperm(T, generator=g) for _ in range(B)]) + 5
    return rank // 7


@pytest.mark.parametrize("kind", ["documents", "shuffled", "coarse"])
def test_forward_loop_with_position_ids_of_the_callers_choosing(emu, monkeypatch, kind):
    """tah_model.py:499 hands position_ids through and :788 compares them as plain numbers: with
    POSITION_IDS_ARE_RANKS off every key carries its position and the loop gives what the dense restatement gives
    with the same ids, over three depths, outputs and gradients."""
    import tah_amd.attention as A
    monkeypatch.setattr(A, "POSITION_IDS_ARE_RANKS", False)
    c = make_dense_case(47, B=2, T=40, p_hard=0.4, Hq=2, Hkv=1, D=128, left_pad=[0, 6])
    ids = caller_position_ids(c, 48, kind)
    outs, leaves, rleaves = _loops_over_depths(c, _deeper_levels(c, 49, 1), requires_grad=True, position_ids=ids)
    check_depth_outputs(c, outs)
    check_depth_gradients(c, outs, leaves, rleaves)


def test_depth_limits(emu):
    """Negative depths are refused; with the decode path's slabs enabled a cache holds two depths and says so."""
    from tah_amd import TahDuoError
    from tah_amd.attention import build_attention_mask
    from tah_amd.cache import TaHDuoCache
    cache = TaHDuoCache()
    pos, one = torch.arange(4)[None], torch.ones(1, 4, dtype=torch.long)
    with pytest.raises(TahDuoError, match="depth"):
        build_attention_mask(pos, one, cache, -1)
    k = torch.zeros(1, 1, 4, 128, dtype=torch.bfloat16)
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = -1, pos, one
    with pytest.raises(TahDuoError, match="depth"):
        cache.update(k, k, 0)
    slabbed = TaHDuoCache().enable_slabs(8, 8)
    slabbed.current_iter_depth, slabbed.position_ids_to_cache, slabbed.valid_mask_to_cache = 2, pos, one
    with pytest.raises(TahDuoError, match="slabs"):
        slabbed.update(k, k, 0)


def test_position_check_switch(emu):
    """CHECK_POSITIONS: positions that are not the valid tokens' ranks are refused (the kernels would use the ranks)."""
    from tah_amd import TahDuoError, attention
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(36, B=2, T=8, p_hard=0.0, Hq=2, Hkv=1, D=128, left_pad=[0, 3])
    bf = lambda x: x.to(torch.bfloat16)
    pos = (torch.cumsum(c["valid"], -1) - 1).clamp(min=0)
    attention.CHECK_POSITIONS = True
    try:
        for shift, ok in ((0, True), (10, False)):
            cache = TaHDuoCache()
            p = pos + shift
            m = attention.build_attention_mask(p, c["valid"], cache, 0)
            cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, p, c["valid"]
            k, v = cache.update(bf(c["k1"]), bf(c["v1"]), 0)
            if ok:
                attention.duo_attention_forward(_layer(), bf(c["q1"]), k, v, m, scaling=c["scale"])
            else:
                with pytest.raises(TahDuoError, match="position"):
                    attention.duo_attention_forward(_layer(), bf(c["q1"]), k, v, m, scaling=c["scale"])
    finally:
        attention.CHECK_POSITIONS = False


def test_forward_loop_without_host_sync(emu):
    """HOST_SYNC = False: prefill (left-padded batch) and a decode step at both depths, packed by upper bounds."""
    from tests.sync_free_case import run
    assert run("cpu", B=2, T=24, left_pad=(0, 7), Hq=2, Hkv=1)


def test_gather_with_max_active_and_overflow_flag(emu):
    from tah_amd.pack import gather_active, scatter_back
    g = torch.Generator().manual_seed(8)
    B, S = 3, 17
    mask = torch.rand(B, S, generator=g) < 0.4
    mask[1] = False
    x = torch.randn(B, S, 4, generator=g).to(torch.bfloat16)
    ids = torch.arange(B * S).view(B, S)
    wpad, wx, wi = O.gather_active(mask, x, ids)
    n = wpad.shape[1]
    pad, gx, gi = gather_active(mask, x, ids, max_active=n + 2)
    assert int(pad.overflow) == 0 and pad.shape == (B, n + 2)
    assert torch.equal(pad[:, :n], wpad) and pad[:, n:].all()
    assert torch.equal(gx[:, :n], wx) and torch.equal(gi[:, :n], wi) and (gx[:, n:] == 0).all()
    dest = torch.full((B, S, 4), -7.0).to(torch.bfloat16)
    assert torch.equal(scatter_back(mask, gx, dest, host_sync=False), O.scatter_back(mask, wx, dest))
    # a width below the busiest row: the surplus is dropped and the flag raised
    pad, gx = gather_active(mask, x, max_active=n - 1)
    assert int(pad.overflow) == 1 and torch.equal(gx, wx[:, : n - 1])
    part = scatter_back(mask, gx, dest, host_sync=False)
    want = O.scatter_back(mask, wx, dest)
    counts = mask.sum(1)
    for b in range(B):
        cols = torch.nonzero(mask[b]).flatten()
        kept = cols[: n - 1]
        assert torch.equal(part[b, kept], want[b, kept])
        if counts[b] == n:
            assert (part[b, cols[-1]] == -7).all()  # the dropped entry's place keeps what dest held


def test_hard_index_of_mask_without_columns(emu):
    """S == 0: every boundary is zero (nothing read from uninitialised memory)."""
    from tah_amd.pack import HardIndex, gather_active
    idx = HardIndex(torch.zeros(3, 0, dtype=torch.bool))
    assert idx.cu.tolist() == [0, 0, 0, 0] and idx.n == 0 and idx.width == 0
    pad, x = gather_active(torch.zeros(3, 0, dtype=torch.bool), torch.zeros(3, 0, 4))
    assert pad.shape == (3, 0) and x.shape == (3, 0, 4)


def test_reorder_cache_with_slabs(emu):
    """Beam-search reorder moves slab rows, positions and lengths together (causal_cache.py:201-205 for K/V)."""
    from tests.reorder_case import run
    plain, moved, beam = run("cpu")
    for a, b in zip(plain, moved):
        assert torch.equal(a[beam], b)


def test_reorder_cache_chunks_only():
    """Without slabs: K and V chunks are index-selected along the batch axis, nothing else changes."""
    from tah_amd.cache import TaHDuoCache
    c = TaHDuoCache()
    pos = torch.arange(5)[None].expand(3, 5)
    c.current_iter_depth, c.position_ids_to_cache, c.valid_mask_to_cache = 0, pos, torch.ones(3, 5, dtype=torch.long)
    k, v = torch.randn(3, 2, 5, 8), torch.randn(3, 2, 5, 8)
    c.update(k, v, 0)
    beam = torch.tensor([1, 1, 0])
    c.reorder_cache(beam)
    K, V = c.get_cache_upto_iter(0, 0)
    assert torch.equal(K, k[beam]) and torch.equal(V, v[beam])
    assert torch.equal(c.get_position_id_upto_iter(0, 0), pos)


def test_metadata_getters_leave_the_chunk_lists_alone():
    """The getters fold positions / valid flags of many writes in a memo of their own; the per-write lists that
    chunks() pairs with the K/V chunks keep one entry per write, before and after (and between) getter calls."""
    from tah_amd.attention import _Packed
    from tah_amd.cache import TaHDuoCache
    from tah_amd import TahDuoError
    cache = TaHDuoCache()
    B, H, D = 2, 2, 8
    widths = [4, 1, 3]
    for i, T in enumerate(widths):
        cache.current_iter_depth = 0
        cache.position_ids_to_cache = torch.arange(T).repeat(B, 1) + 10 * i
        cache.valid_mask_to_cache = torch.ones(B, T, dtype=torch.long)
        cache.update(torch.randn(B, H, T, D), torch.randn(B, H, T, D), 0)
        pos = cache.get_position_id_upto_iter(0, 0)
        assert pos.shape == (B, sum(widths[: i + 1]))
        assert cache.get_valid_mask_upto_iter(0, 0).shape == pos.shape
    want = torch.cat([torch.arange(T).repeat(B, 1) + 10 * i for i, T in enumerate(widths)], dim=-1)
    assert torch.equal(cache.get_position_id_upto_iter(0, 0), want)
    ch = cache.chunks(0, 0)
    assert len(ch) == len(widths)
    for (k, v, pos, valid), T in zip(ch, widths):
        assert k.shape[-2] == v.shape[-2] == pos.shape[-1] == valid.shape[-1] == T
    with pytest.raises(TahDuoError):  # a valid mask of another width than the block it is said to describe
        _Packed(torch.ones(B, 5, dtype=torch.long), None, B, 4, torch.device("cpu"))
