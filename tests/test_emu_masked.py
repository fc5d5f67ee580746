"""Additive-mask compatibility mode (forward and backward kernels) on the CPU execution shim against the
oracle's restatement of mask + SDPA.  No GPU."""
import numpy as np
import pytest
import torch

from oracle import duo_oracle as O
from tests import emu_util
from tests.cases import make_masked_case

pytestmark = pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")


def _reference(case, d_o=None):
    """float64 SDPA with the additive mask; with d_o also dq, dk, dv by autograd."""
    q, k, v = (case[n].double().requires_grad_(d_o is not None) for n in ("q", "k", "v"))
    o = O.sdpa_dense(q, k, v, case["mask"].double(), case["scale"])
    if d_o is None:
        return o.detach()
    o.backward(d_o.double())
    return o.detach(), q.grad, k.grad, v.grad


@pytest.mark.parametrize("hq,hkv,B,tq,tk,mdt,per_head", [
    (2, 1, 2, 40, 70, torch.float32, False),    # G=2, (B,1,Tq,Tkv) fp32 mask, ragged tile
    (2, 2, 1, 130, 130, torch.bfloat16, False),  # G=1, bf16 mask, two query tiles
    (4, 1, 2, 9, 65, torch.float32, True),      # G=4, per-head mask
])
def test_masked_forward_and_backward_on_cpu_shim(hq, hkv, B, tq, tk, mdt, per_head):
    from tah_amd import attention
    case = make_masked_case(50 + hq, B, hq, hkv, tq, tk, mask_dtype=mdt, per_head=per_head)
    g = torch.Generator().manual_seed(3)
    d_o = torch.randn(B, tq, hq, 128, generator=g).to(torch.bfloat16)
    # Row 0 of the last batch entry hides every key: SDPA then averages V over the finfo.min entries
    # (garbage the reference discards, so no gradient comes back through it); the kernels return zeros.
    d_o[B - 1, 0] = 0
    want_o, want_dq, want_dk, want_dv = _reference(case, d_o.float())
    want_o[B - 1, 0] = 0
    q, k, v = (case[n].clone().requires_grad_(True) for n in ("q", "k", "v"))
    with emu_util.emulated():
        o, lse = attention.attn_additive_mask(q, k, v, case["mask"], case["scale"], return_lse=True)
        o.backward(d_o)
    np.testing.assert_allclose(o.detach().float().numpy(), want_o.numpy(), atol=2e-2, rtol=2e-2)
    # log-sum-exp against the same float64 scores
    s = torch.matmul(case["q"].double(), O.repeat_kv(case["k"].double(), hq // hkv).transpose(-1, -2)) * case["scale"]
    want_lse = torch.logsumexp(s + case["mask"].double(), dim=-1)          # (B,Hq,Tq)
    got_lse = lse.view(hq, B, tq).permute(1, 0, 2)
    vis = torch.isfinite(want_lse) & (want_lse > -1e30)
    np.testing.assert_allclose(got_lse[vis].numpy(), want_lse[vis].numpy(), atol=2e-3, rtol=1e-3)
    for name, got, want in (("dq", q.grad, want_dq), ("dk", k.grad, want_dk), ("dv", v.grad, want_dv)):
        d = (got.double() - want).abs()
        ma, mr = d.max() / want.abs().max(), d.mean() / want.abs().mean()
        assert ma <= 2e-2 and mr <= 1e-2, f"{name}: max-err/max|ref| {ma:.3e}, mean-rel-err {mr:.3e}"


def test_masked_mode_equals_duo_kernel_on_the_reference_mask():
    """The dense mask the reference would build for a depth-0 prefill (plain causal + left padding) gives, in
    compatibility mode, what the duo-causal entry point gives from positions alone."""
    from tah_amd import attention, ops
    B, T, hq, hkv = 2, 70, 2, 1
    case = make_masked_case(77, B, hq, hkv, T, T, mask_dtype=torch.float32)
    pos = torch.arange(T)
    mask = torch.where(pos[None, :] <= pos[:, None], 0.0, torch.finfo(torch.float32).min)[None, None].expand(B, 1, T, T).contiguous()
    with emu_util.emulated():
        o_mask = attention.attn_additive_mask(case["q"], case["k"], case["v"], mask, case["scale"])
        rows = lambda x: x.transpose(1, 2).reshape(B * T, x.shape[1], 128)
        cu = torch.arange(0, (B + 1) * T, T, dtype=torch.int32)
        z, zi = torch.zeros(B + 1, dtype=torch.int32), torch.zeros(0, dtype=torch.int32)
        q, k, v = rows(case["q"]), rows(case["k"]), rows(case["v"])
        o_duo = ops.duo_fwd_varlen(q, k, v, cu, cu, q[:0], k[:0], v[:0], zi, zi, z, z, case["scale"])[0]
    np.testing.assert_allclose(o_mask.reshape(B * T, hq, 128).float().numpy(), o_duo.float().numpy(), atol=4e-3, rtol=4e-3)
