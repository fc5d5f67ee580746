"""Pins oracle/qk_prep_ref.py: against the installed transformers' Qwen3RMSNorm / apply_rotary_pos_emb
(bf16 on the CPU) and against what the mathematics fixes.  No GPU."""
import numpy as np
import pytest
import torch

from oracle import qk_prep_ref as R


def _bf(x):
    return torch.from_numpy(np.ascontiguousarray(x)).to(torch.bfloat16)


def _case(seed, rows=37, hq=4, hkv=2, d=128, scale=1.0):
    g = np.random.default_rng(seed)
    rb = lambda *s: R.bf16_round((g.standard_normal(s) * scale).astype(np.float32))
    q, k = rb(rows, hq, d), rb(rows, hkv, d)
    qw, kw = R.bf16_round((1.0 + 0.2 * g.standard_normal(d)).astype(np.float32)), R.bf16_round((1.0 + 0.2 * g.standard_normal(d)).astype(np.float32))
    cos, sin = R.rotary_tables(g.integers(0, 40000, rows))
    return q, k, qw, kw, cos, sin


def test_bf16_round_matches_torch():
    g = np.random.default_rng(0)
    x = np.concatenate([g.standard_normal(5000).astype(np.float32) * 10.0 ** g.integers(-20, 20, 5000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(R.bf16_round(x), want)


@pytest.mark.parametrize("seed,scale", [(1, 1.0), (2, 0.05), (3, 30.0)])
def test_against_transformers_modules(seed, scale):
    m = pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    q, k, qw, kw, cos, sin = _case(seed, scale=scale)
    eps = 1e-6
    qn, kn = m.Qwen3RMSNorm(128, eps=eps).to(torch.bfloat16), m.Qwen3RMSNorm(128, eps=eps).to(torch.bfloat16)
    with torch.no_grad():
        qn.weight.copy_(_bf(qw)), kn.weight.copy_(_bf(kw))
        # (rows, H, D) -> (1, H, rows, D), the layout apply_rotary_pos_emb is called with
        tq, tk = qn(_bf(q)).transpose(0, 1)[None], kn(_bf(k)).transpose(0, 1)[None]
        wq, wk = m.apply_rotary_pos_emb(tq, tk, _bf(cos)[None], _bf(sin)[None])
    wq, wk = wq[0].transpose(0, 1).float().numpy(), wk[0].transpose(0, 1).float().numpy()
    gq, gk = R.qk_prep(q, k, qw, kw, cos, sin, eps)
    for got, want in ((gq, wq), (gk, wk)):
        exact = np.mean(got == want)
        ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64)) >> 16
        assert exact > 0.999 and ulp.max() <= 1, (exact, ulp.max())


def test_unit_weights_give_unit_rms_and_position_zero_is_identity():
    q, k, _, _, _, _ = _case(4)
    one = np.ones(128, np.float32)
    n = R.rms_norm(q, one, 1e-6)
    np.testing.assert_allclose(np.sqrt(np.mean(n.astype(np.float64) ** 2, -1)), 1.0, atol=4e-3)
    cos, sin = R.rotary_tables(np.zeros(q.shape[0], np.int64))
    np.testing.assert_array_equal(R.rope(n, cos, sin), n)


def test_rotation_keeps_pair_norms_and_composes():
    q, _, qw, _, cos, sin = _case(5)
    y = R.rms_norm(q, qw, 1e-6)
    o = R.rope(y, cos, sin)
    pair = lambda t: t[..., :64].astype(np.float64) ** 2 + t[..., 64:].astype(np.float64) ** 2
    np.testing.assert_allclose(pair(o), pair(y), rtol=0.03, atol=2e-3)
    # against the textbook complex rotation in float64, on the un-rounded tables' bf16 values
    z = (y[..., :64] + 1j * y[..., 64:]) * (cos[:, None, :64] + 1j * sin[:, None, :64])
    np.testing.assert_allclose(o[..., :64], z.real, atol=0.03, rtol=0.02)
    np.testing.assert_allclose(o[..., 64:], z.imag, atol=0.03, rtol=0.02)


def test_backward_against_autograd_through_the_transformers_modules_and_finite_differences():
    m = pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    q, k, qw, kw, cos, sin = _case(7, rows=9, hq=4, hkv=2, scale=2.0)
    eps = 1e-6
    g = np.random.default_rng(8)
    gq, gk = g.standard_normal(q.shape), g.standard_normal(k.shape)
    qn, kn = m.Qwen3RMSNorm(128, eps=eps).double(), m.Qwen3RMSNorm(128, eps=eps).double()
    with torch.no_grad():
        qn.weight.copy_(torch.from_numpy(qw).double()), kn.weight.copy_(torch.from_numpy(kw).double())
    tq, tk = torch.from_numpy(q).double().requires_grad_(True), torch.from_numpy(k).double().requires_grad_(True)
    oq, ok = m.apply_rotary_pos_emb(qn(tq).transpose(0, 1)[None], kn(tk).transpose(0, 1)[None],
                                    torch.from_numpy(cos).double()[None], torch.from_numpy(sin).double()[None])
    loss = (oq[0].transpose(0, 1) * torch.from_numpy(gq)).sum() + (ok[0].transpose(0, 1) * torch.from_numpy(gk)).sum()
    loss.backward()
    dq, dk, dqw, dkw = R.qk_prep_backward(q, k, qw, kw, cos, sin, eps, gq, gk)
    # (Qwen3RMSNorm computes in float32 whatever it is given: its gradients carry float32 rounding)
    for got, want in ((dq, tq.grad), (dk, tk.grad), (dqw, qn.weight.grad), (dkw, kn.weight.grad)):
        np.testing.assert_allclose(got, want.numpy(), rtol=2e-4, atol=2e-5 * float(np.abs(got).max()))
    # and one entry of each by central differences of the real-valued forward
    def f(qx, qwx):
        x = qx.astype(np.float64)
        y = qwx.astype(np.float64) * x / np.sqrt(np.mean(x * x, -1, keepdims=True) + eps)
        rot = np.concatenate([-y[..., 64:], y[..., :64]], -1)
        return ((y * cos[:, None, :].astype(np.float64) + rot * sin[:, None, :].astype(np.float64)) * gq).sum()
    h = 1e-5
    e = np.zeros_like(q, dtype=np.float64); e[3, 1, 70] = h
    assert abs((f(q + e, qw) - f(q - e, qw)) / (2 * h) - dq[3, 1, 70]) < 1e-6 * max(1.0, abs(dq[3, 1, 70]))
    ew = np.zeros(128); ew[5] = h
    assert abs((f(q, qw + ew) - f(q, qw - ew)) / (2 * h) - dqw[5]) < 1e-6 * max(1.0, abs(dqw[5]))
