"""GPU parity of the q/k RMSNorm + rotary embedding (+ KV append) kernel through the C ABI vs the oracle."""
import numpy as np
import pytest
import torch

from oracle import qk_prep_ref as R
from tests.qk_prep_cases import assert_bf16_close, make_case, to_torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,hq,hkv,scale,seed", [
    (512, 16, 8, 1.0, 1),      # Qwen3-1.7B head shape
    (1000, 16, 8, 25.0, 2),    # large activations
    (77, 8, 1, 0.02, 3),       # small activations (eps matters), group of 8
    (1, 4, 4, 1.0, 4),         # one decode row
    (65, 32, 8, 1.0, 8),       # 48 head slots per row: three passes
])
def test_norm_rope_matches_oracle(rows, hq, hkv, scale, seed):
    from tah_amd.kv_cache import qk_norm_rope
    print(f"case qk_prep rows={rows} hq={hq} hkv={hkv} scale={scale} seed={seed}", flush=True)
    c = make_case(seed, rows, hq, hkv, scale=scale)
    t = to_torch(c, "cuda")
    q_out, k_out = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"])
    torch.cuda.synchronize()
    wq, wk = R.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    print("exact fractions", assert_bf16_close(q_out, wq, "q"), assert_bf16_close(k_out, wk, "k"), flush=True)


def test_matches_the_installed_transformers_modules_on_the_gpu():
    """The same tensors through transformers' own Qwen3RMSNorm / apply_rotary_pos_emb in bf16 on the device."""
    m = pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    from tah_amd.kv_cache import qk_norm_rope
    c = make_case(5, 300, 16, 8)
    t = to_torch(c, "cuda")
    q_out, k_out = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"])
    qn = m.Qwen3RMSNorm(128, eps=c["eps"]).to("cuda", torch.bfloat16)
    kn = m.Qwen3RMSNorm(128, eps=c["eps"]).to("cuda", torch.bfloat16)
    with torch.no_grad():
        qn.weight.copy_(t["qw"]), kn.weight.copy_(t["kw"])
        tq, tk = qn(t["q"]).transpose(0, 1)[None], kn(t["k"]).transpose(0, 1)[None]
        wq, wk = m.apply_rotary_pos_emb(tq, tk, t["cos"][None], t["sin"][None])
    assert_bf16_close(q_out, wq[0].transpose(0, 1).float().cpu().numpy(), "q vs transformers")
    assert_bf16_close(k_out, wk[0].transpose(0, 1).float().cpu().numpy(), "k vs transformers")


def test_fused_append_equals_norm_rope_then_append_full_prefill_shape():
    from tah_amd.kv_cache import KvSlabs, qk_norm_rope
    B, T = 4, 4096
    c = make_case(6, B * T, 16, 8, scale=0.5, max_pos=T)
    t = to_torch(c, "cuda")
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    a, b = KvSlabs(B, T, 8, with_pos=True, device="cuda"), KvSlabs(B, T, 8, with_pos=True, device="cuda")
    q1, none = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], v=t["v"], cache=a, cu_new=cu,
                            pos_new=t["pos"])
    q2, k2 = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"])
    b.append(k2, t["v"], cu, pos_new=t["pos"])
    torch.cuda.synchronize()
    assert none is None and torch.equal(q1, q2)
    for x, y in ((a.k, b.k), (a.v, b.v), (a.pos, b.pos), (a.len, b.len)):
        assert torch.equal(x, y)
    assert a.len.tolist() == [T] * B and a.overflow.item() == 0
    wq, _ = R.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    assert_bf16_close(q1, wq, "q full size")


def test_in_place_and_overflow():
    from tah_amd.kv_cache import KvSlabs, qk_norm_rope
    c = make_case(7, 40, 16, 8)
    t = to_torch(c, "cuda")
    fused = torch.zeros(40, 32, 128, dtype=torch.bfloat16, device="cuda")
    fused[:, :16], fused[:, 16:24], fused[:, 24:] = t["q"], t["k"], t["v"]
    qk_norm_rope(fused[:, :16], fused[:, 16:24], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], in_place=True)
    wq, wk = R.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    assert_bf16_close(fused[:, :16], wq, "q in place")
    assert_bf16_close(fused[:, 16:24], wk, "k in place")
    assert torch.equal(fused[:, 24:], t["v"])
    s = KvSlabs(2, 16, 8, with_pos=False, device="cuda")
    qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], v=t["v"], cache=s,
                 cu_new=torch.tensor([0, 10, 40], dtype=torch.int32, device="cuda"))
    torch.cuda.synchronize()
    assert s.len.tolist() == [10, 16] and s.overflow.item() == 1


def test_input_norm_folded_in_equals_scaling_the_projections_first_gpu():
    from tah_amd.kv_cache import qk_norm_rope
    from tests.qk_prep_cases import folded_norm_case
    c, t, x, wq, wk, wv = folded_norm_case("cuda", seed=61, rows=300, hq=16, hkv=8, hidden=2048)
    q_out, k_out, v_out = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], v=t["v"],
                                       norm_input=x, norm_eps=1e-6)
    assert_bf16_close(q_out, wq, "q")
    assert_bf16_close(k_out, wk, "k")
    assert float((v_out.float().cpu() == torch.from_numpy(wv)).float().mean()) >= 0.99
    assert torch.allclose(v_out.float().cpu(), torch.from_numpy(wv), rtol=2 ** -7, atol=0)



@pytest.mark.parametrize("rows,hq,hkv,scale,n_partial", [(1000, 16, 8, 1.0, None), (16384, 16, 8, 1.0, None), (77, 4, 4, 15.0, 16), (5, 32, 8, 0.05, 64)])
def test_backward_matches_analytic_gradients_gpu(rows, hq, hkv, scale, n_partial):
    from tests.qk_prep_cases import check_backward
    check_backward("cuda", 90 + hq, rows, hq, hkv, scale=scale, n_partial=n_partial)
