"""GPU: the host layer (pack API, cache, mask carrier, HF attention callable) end to end on the HIP path."""
import numpy as np
import pytest
import torch

from oracle import duo_oracle as O
from tests.cases import make_dense_case
from tests.test_host_layer import (_deeper_levels, caller_position_ids, _forward_two_depths, _forward_two_depths_reference_style, _loops_over_depths,
                                   _oracle_two_depths, check_depth_gradients, check_depth_outputs)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,T,p,left_pad", [(2, 300, 0.1, None), (3, 200, 0.2, [0, 37, 150]), (1, 512, 0.06, None), (2, 2300, 0.1, [0, 700])])
def test_forward_loop_matches_dense_reference_gpu(B, T, p, left_pad):
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(50 + B, B=B, T=T, p_hard=p, left_pad=left_pad)
    _, o1, o2, pad = _forward_two_depths(c, TaHDuoCache(), device="cuda")
    w1, w2, wpad = _oracle_two_depths(c)
    assert torch.equal(pad.cpu(), wpad)
    valid = c["valid"].bool()
    np.testing.assert_allclose(o1.cpu()[valid].float().numpy(), w1[valid].numpy(), atol=2e-2, rtol=2e-2)
    assert (o1.cpu()[~valid] == 0).all()
    np.testing.assert_allclose(o2.cpu()[~pad.cpu()].float().numpy(), w2[~wpad].numpy(), atol=2e-2, rtol=2e-2)


def test_reference_style_loop_with_dense_masks_gpu():
    """Additive-mask compatibility mode end to end: dense masks + concatenated cache give what the symbolic
    mask carrier gives (and what the dense oracle gives) on every valid row."""
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(51, B=3, T=200, p_hard=0.2, left_pad=[0, 37, 150])
    o1, o2, pad = _forward_two_depths_reference_style(c, TaHDuoCache(), device="cuda")
    _, d1, d2, _ = _forward_two_depths(c, TaHDuoCache(), device="cuda")
    w1, w2, wpad = _oracle_two_depths(c)
    valid = c["valid"].bool()
    np.testing.assert_allclose(o1.cpu()[valid].float().numpy(), w1[valid].numpy(), atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(o2.cpu()[~pad.cpu()].float().numpy(), w2[~wpad].numpy(), atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(o1.cpu()[valid].float().numpy(), d1.cpu()[valid].float().numpy(), atol=8e-3, rtol=8e-3)
    np.testing.assert_allclose(o2.cpu()[~pad.cpu()].float().numpy(), d2.cpu()[~pad.cpu()].float().numpy(), atol=8e-3, rtol=8e-3)


def test_forward_loop_gradients_gpu():
    from tah_amd.cache import TaHDuoCache
    c = make_dense_case(60, B=2, T=160, p_hard=0.2, left_pad=[0, 30])
    t, o1, o2, pad = _forward_two_depths(c, TaHDuoCache(), requires_grad=True, device="cuda")
    g = torch.Generator().manual_seed(1)
    w1, w2 = torch.randn(o1.shape, generator=g), torch.randn(o2.shape, generator=g)
    ((o1.float() * w1.cuda()).sum() + (o2.float() * w2.cuda()).sum()).backward()
    ref = {k: c[k].to(torch.bfloat16).double().requires_grad_(True) for k in t}
    r1, r2, rpad = O.duo_prefill_dense(ref["q1"], ref["k1"], ref["v1"], ref["q2"], ref["k2"], ref["v2"], c["hard"],
                                       c["scale"], valid_mask=c["valid"])
    valid = c["valid"].bool()
    # invalid query rows are out of contract: they take no part in the loss
    ((r1 * (w1 * valid[:, :, None, None]).to(torch.bfloat16).double()).sum()
     + (r2 * (w2 * ~rpad[:, :, None, None]).to(torch.bfloat16).double()).sum()).backward()
    for n in ("q1", "k1", "v1", "q2", "k2", "v2"):
        a, b = t[n].grad.float().cpu(), ref[n].grad.float()
        err = (a - b).abs().max() / b.abs().max()
        assert err < 3e-2, (n, float(err))


def test_gather_scatter_large_gpu():
    from tah_amd.pack import gather_active, scatter_back
    g = torch.Generator().manual_seed(7)
    B, S, H = 4, 4096, 2048
    mask = (torch.rand(B, S, generator=g) < 0.06).cuda()
    x = torch.randn(B, S, H, generator=g).to(torch.bfloat16).cuda()
    pos = torch.arange(S).expand(B, S).contiguous().cuda()
    pad, gx, gp = gather_active(mask, x, pos)
    assert torch.equal(gx[~pad], x[mask]) and torch.equal(gp[~pad], pos[mask])
    assert (gx[pad] == 0).all() and pad.shape[1] == int(mask.sum(1).max())
    dest = torch.zeros_like(x)
    out = scatter_back(mask, gx, dest)
    assert torch.equal(out[mask], x[mask]) and (out[~mask] == 0).all()


def test_reorder_cache_with_slabs_gpu():
    from tests.reorder_case import run
    plain, moved, beam = run("cuda", beam=(3, 0, 0, 2), T0=70)
    for a, b in zip(plain, moved):
        assert torch.equal(a[beam], b)


def test_decode_steps_both_depths_through_cache_and_callable_gpu():
    """Prefill + decode steps at depth 0 and depth 1 (hard subset, pad rows, left padding, slabs on) through
    TaHDuoCache + duo_attention_forward on the device, against the concatenating oracle cache + dense SDPA
    (tah_model.py:116-118 pad rows, causal_cache.py:84-97 depth-1 appends for all B rows)."""
    from tests.decode_steps_case import run
    cache, n1 = run("cuda", T0=150, steps=5, B=3, left_pad=(0, 37, 9), seed=61, Hq=16, Hkv=8,
                    force_hard=[[0], [], [0, 1, 2], [2], [1]])
    assert n1 == 4
    from tah_amd import TahDuoError
    with pytest.raises(TahDuoError):
        cache.get_cache_upto_iter(0, 0)


def test_slab_overflow_raises_gpu():
    from tah_amd import TahDuoError
    from tah_amd.cache import TaHDuoCache
    cache = TaHDuoCache().enable_slabs(4, 4)
    k = torch.zeros(2, 8, 3, 128, dtype=torch.bfloat16, device="cuda")
    pos, one = torch.arange(3, device="cuda")[None].expand(2, 3), torch.ones(2, 3, dtype=torch.long, device="cuda")
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, one
    cache.update(k, k, 0)
    with pytest.raises(TahDuoError, match="capacity"):
        cache.update(k, k, 0)


def test_forward_loop_without_host_sync_gpu():
    """Prefill + a decode step at both depths through the host layer with no host synchronisation at all
    (torch.cuda.set_sync_debug_mode("error") is on while the loop runs; tah_model.py:116, 580 are the syncs the
    reference's loop has there)."""
    from tests.sync_free_case import run
    assert run("cuda", B=3, T=300, p=0.1, left_pad=(0, 37, 150), Hq=16, Hkv=8)


@pytest.mark.parametrize("B,T,p,left_pad,n_deeper", [(2, 300, 0.3, [0, 41], 1), (1, 600, 0.25, None, 2)])
def test_forward_loop_over_more_than_two_depths_gpu(B, T, p, left_pad, n_deeper):
    """Latent depths 2 and 3 (tah_model.py:788 takes any): outputs and gradients against the dense restatement."""
    c = make_dense_case(70 + B, B=B, T=T, p_hard=p, left_pad=left_pad)
    deeper = _deeper_levels(c, 71, n_deeper)
    outs, leaves, rleaves = _loops_over_depths(c, deeper, requires_grad=True, device="cuda")
    check_depth_outputs(c, outs)
    check_depth_gradients(c, outs, leaves, rleaves)


@pytest.mark.parametrize("kind", ["documents", "shuffled"])
def test_forward_loop_with_position_ids_of_the_callers_choosing_gpu(monkeypatch, kind):
    """POSITION_IDS_ARE_RANKS off: every key carries its position (tah_model.py:499, :788 with plain numbers)."""
    import tah_amd.attention as A
    monkeypatch.setattr(A, "POSITION_IDS_ARE_RANKS", False)
    c = make_dense_case(80, B=2, T=330, p_hard=0.3, left_pad=[0, 50])
    ids = caller_position_ids(c, 81, kind)
    outs, leaves, rleaves = _loops_over_depths(c, _deeper_levels(c, 82, 1), requires_grad=True, device="cuda", position_ids=ids)
    check_depth_outputs(c, outs)
    check_depth_gradients(c, outs, leaves, rleaves)
