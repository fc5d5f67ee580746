"""GPU parity of the additive-mask compatibility mode (forward and backward through the C ABI) against the
oracle's float64 restatement of mask + SDPA."""
import numpy as np
import pytest
import torch

from oracle import duo_oracle as O
from tests.cases import make_masked_case
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("hq,hkv,B,tq,tk,mdt,per_head", [
    (16, 8, 2, 300, 500, torch.bfloat16, False),  # the reference's (B,1,Tq,Tkv) bf16 mask, Tkv > Tq (cached keys)
    (16, 8, 1, 512, 512, torch.float32, False),   # BASELINE config 0 shape, fp32 mask
    (8, 2, 2, 70, 129, torch.float32, True),      # group of 4, per-head mask, ragged tiles
    (8, 1, 1, 33, 64, torch.bfloat16, False),     # group of 8
])
def test_masked_fwd_bwd_match_oracle(hq, hkv, B, tq, tk, mdt, per_head):
    from tah_amd import attention
    print(f"case masked hq={hq} hkv={hkv} B={B} tq={tq} tk={tk} {mdt} per_head={per_head}", flush=True)
    case = make_masked_case(90 + hq, B, hq, hkv, tq, tk, mask_dtype=mdt, per_head=per_head)
    g = torch.Generator().manual_seed(5)
    d_o = torch.randn(B, tq, hq, 128, generator=g).to(torch.bfloat16)
    d_o[B - 1, 0] = 0  # the row that hides every key takes no part (the reference discards it)
    qr, kr, vr = (case[n].double().requires_grad_(True) for n in ("q", "k", "v"))
    want = O.sdpa_dense(qr, kr, vr, case["mask"].double(), case["scale"])
    want.backward(d_o.double())
    want = want.detach()
    want[B - 1, 0] = 0
    q, k, v = (case[n].cuda().requires_grad_(True) for n in ("q", "k", "v"))
    o = attention.attn_additive_mask(q, k, v, case["mask"].cuda(), case["scale"])
    o.backward(d_o.cuda())
    torch.cuda.synchronize()
    print("o", assert_close(o.detach(), want.float().numpy(), "masked o"), flush=True)
    for name, got, ref in (("dq", q.grad, qr.grad), ("dk", k.grad, kr.grad), ("dv", v.grad, vr.grad)):
        d = (got.double().cpu() - ref).abs()
        ma, mr = float(d.max() / ref.abs().max()), float(d.mean() / ref.abs().mean())
        print(name, ma, mr, flush=True)
        # same bars as the duo-causal gradients: max-err / max|ref| <= 2e-2, mean relative error <= 1e-2
        assert ma <= 2e-2 and mr <= 1e-2, f"{name}: max-err/max|ref| {ma:.3e}, mean-rel-err {mr:.3e}"


def test_masked_rejects_bad_inputs():
    from tah_amd import TahDuoError, attention
    case = make_masked_case(1, 1, 2, 1, 8, 8)
    q, k, v, m = (case[n].cuda() for n in ("q", "k", "v", "mask"))
    with pytest.raises(TahDuoError):
        attention.attn_additive_mask(q, k, v, m[..., :7], case["scale"])          # mask narrower than the keys
    with pytest.raises(TahDuoError):
        attention.attn_additive_mask(q, k, v, m.to(torch.float16), case["scale"])  # unsupported mask dtype
