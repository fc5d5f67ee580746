"""Shared input builder and checks for the q/k RMSNorm + rotary (+ append) tests."""
import numpy as np
import torch

from oracle import qk_prep_ref as R


def make_case(seed, rows, hq, hkv, d=128, scale=1.0, max_pos=40000):
    g = np.random.default_rng(seed)
    rb = lambda *s: R.bf16_round((g.standard_normal(s) * scale).astype(np.float32))
    pos = g.integers(0, max_pos, rows)
    cos, sin = R.rotary_tables(pos)
    return dict(q=rb(rows, hq, d), k=rb(rows, hkv, d), v=rb(rows, hkv, d),
                qw=R.bf16_round((1.0 + 0.2 * g.standard_normal(d)).astype(np.float32)),
                kw=R.bf16_round((1.0 + 0.2 * g.standard_normal(d)).astype(np.float32)),
                cos=cos, sin=sin, pos=pos.astype(np.int32), eps=1e-6)


def to_torch(case, device):
    return {k: (torch.from_numpy(v).to(torch.bfloat16).to(device) if isinstance(v, np.ndarray) and v.dtype == np.float32
                else (torch.from_numpy(v).to(device) if isinstance(v, np.ndarray) else v)) for k, v in case.items()}


def assert_bf16_close(got: torch.Tensor, want: np.ndarray, what: str):
    """The kernel and the oracle round at the same places; what is left is the summation order of the
    mean and the reciprocal square root, i.e. one bf16 unit in the last place of a normalised value
    now and then.  The rotation adds two products that may cancel, so the bound is stated against the
    size of the rotary pair (which the rotation keeps), not of the element: error <= 2^-6 of it, and
    all but a few elements equal bit for bit."""
    g = got.float().cpu().numpy()
    half = want.shape[-1] // 2
    mag = np.sqrt(want[..., :half].astype(np.float64) ** 2 + want[..., half:].astype(np.float64) ** 2)
    mag = np.concatenate([mag, mag], axis=-1)
    err = np.abs(g.astype(np.float64) - want)
    exact = float(np.mean(g == want))
    worst = float(np.max(err / np.maximum(mag, 1e-30)))
    assert worst <= 2.0 ** -6 and exact >= 0.995, f"{what}: worst error / pair size {worst:.3e}, exact fraction {exact:.5f}"
    return exact


def folded_norm_case(device, seed=50, rows=6, hq=4, hkv=2, hidden=512):
    """Inputs for the input-norm-folded form and what the plain form gives on explicitly scaled projections:
    returns (tensors, x, want_q, want_k, want_v) with want_* from the oracle on bf16(projection * r),
    r = rsqrt(mean(x^2) + eps) per row."""
    c = make_case(seed, rows, hq, hkv, scale=4.0)
    g = np.random.default_rng(seed + 1)
    x = R.bf16_round((g.standard_normal((rows, hidden)) * 7.0).astype(np.float32))
    r = 1.0 / np.sqrt((x.astype(np.float64) ** 2).mean(-1) + 1e-6)
    sc = lambda a: R.bf16_round((a.astype(np.float64) * r[:, None, None]).astype(np.float32))
    wq, wk = R.qk_prep(sc(c["q"]), sc(c["k"]), c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    t = to_torch(c, device)
    return c, t, torch.from_numpy(x).to(torch.bfloat16).to(device), wq, wk, sc(c["v"])



def check_backward(device, seed, rows, hq, hkv, scale=1.0, n_partial=None):
    """``qk_norm_rope`` under autograd (``tah_qk_prep_bwd``) against the analytic float64 gradients of the oracle.  The
    kernel differentiates in float32 and rounds dq / dk to bf16: error <= 2^-6 of the largest gradient entry of the
    same head (the RMSNorm's projection couples a head's entries) and <= 1 % of the weight gradients' largest entry."""
    from tah_amd import kv_cache
    c = make_case(seed, rows, hq, hkv, scale=scale)
    t = to_torch(c, device)
    g = np.random.default_rng(seed + 1)
    gq = R.bf16_round(g.standard_normal(c["q"].shape).astype(np.float32))
    gk = R.bf16_round(g.standard_normal(c["k"].shape).astype(np.float32))
    leaves = [t[n].clone().requires_grad_(True) for n in ("q", "k", "qw", "kw")]
    if n_partial is not None:
        old, kv_cache._QkNormRope.BWD_PARTIALS = kv_cache._QkNormRope.BWD_PARTIALS, n_partial
    try:
        q_out, k_out = kv_cache.qk_norm_rope(leaves[0], leaves[1], leaves[2], leaves[3], t["cos"], t["sin"], c["eps"])
        wq, wk = R.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
        assert_bf16_close(q_out.detach(), wq, "q")
        assert_bf16_close(k_out.detach(), wk, "k")
        tg = lambda x: torch.from_numpy(x).to(torch.bfloat16).to(device)
        torch.autograd.backward([q_out, k_out], [tg(gq), tg(gk)])
    finally:
        if n_partial is not None:
            kv_cache._QkNormRope.BWD_PARTIALS = old
    want = R.qk_prep_backward(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"], gq, gk)
    for name, leaf, w in zip(("dq", "dk"), leaves[:2], want[:2]):
        got = leaf.grad.float().cpu().numpy().astype(np.float64)
        bound = np.abs(w).max(axis=-1, keepdims=True) * 2.0 ** -6 + 1e-30
        assert (np.abs(got - w) <= bound).all(), f"{name}: worst error / head maximum {float((np.abs(got - w) / bound).max()) * 2.0 ** -6:.3e}"
    for name, leaf, w in zip(("dq_weight", "dk_weight"), leaves[2:], want[2:]):
        got = leaf.grad.float().cpu().numpy().astype(np.float64)
        assert np.abs(got - w).max() <= 1e-2 * np.abs(w).max(), f"{name}: {np.abs(got - w).max() / np.abs(w).max():.3e}"
