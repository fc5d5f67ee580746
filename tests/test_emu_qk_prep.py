"""q/k RMSNorm + rotary embedding (+ KV append) kernel on the CPU execution shim against the oracle.  No GPU."""
import numpy as np
import pytest
import torch

from oracle import qk_prep_ref as R
from tests import emu_util
from tests.qk_prep_cases import assert_bf16_close, make_case, to_torch

pytestmark = pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")


@pytest.mark.parametrize("rows,hq,hkv,scale", [(5, 4, 2, 1.0), (3, 2, 2, 20.0), (4, 8, 1, 0.03), (7, 4, 2, 1.0), (12, 2, 2, 5.0)])
def test_norm_rope_matches_oracle(rows, hq, hkv, scale):
    from tah_amd.kv_cache import qk_norm_rope
    c = make_case(10 + rows, rows, hq, hkv, scale=scale)
    t = to_torch(c, "cpu")
    with emu_util.emulated():
        q_out, k_out = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"])
    wq, wk = R.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    assert_bf16_close(q_out, wq, "q")
    assert_bf16_close(k_out, wk, "k")


def test_input_norm_folded_in_equals_scaling_the_projections_first():
    from tah_amd.kv_cache import KvSlabs, qk_norm_rope
    from tests.qk_prep_cases import folded_norm_case
    c, t, x, wq, wk, wv = folded_norm_case("cpu")
    with emu_util.emulated():
        q_out, k_out, v_out = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], v=t["v"],
                                           norm_input=x, norm_eps=1e-6)
        # and on the way into the slabs
        rows = t["q"].shape[0]
        slabs = KvSlabs(1, rows + 2, t["k"].shape[1], with_pos=False, device="cpu")
        cu = torch.tensor([0, rows], dtype=torch.int32)
        q2, _ = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], v=t["v"], cache=slabs, cu_new=cu,
                             norm_input=x, norm_eps=1e-6)
    assert_bf16_close(q_out, wq, "q")
    assert_bf16_close(k_out, wk, "k")
    assert float((v_out.float() == torch.from_numpy(wv)).float().mean()) >= 0.99  # one bf16 step where r's last bit differs
    assert torch.allclose(v_out.float(), torch.from_numpy(wv), rtol=2 ** -7, atol=0)
    assert torch.equal(q2, q_out)
    assert torch.equal(slabs.k[0, :, :rows].transpose(0, 1), k_out) and torch.equal(slabs.v[0, :, :rows].transpose(0, 1), v_out)


def test_more_heads_than_one_pass_pair_and_empty_input():
    """48 head slots per row (three passes of 16; the first two are loaded up front), and a call with no rows."""
    from tah_amd.kv_cache import qk_norm_rope
    c = make_case(31, 3, 32, 8)
    t = to_torch(c, "cpu")
    with emu_util.emulated():
        q_out, k_out = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"])
        e_q, e_k = qk_norm_rope(t["q"][:0], t["k"][:0], t["qw"], t["kw"], t["cos"][:0], t["sin"][:0], c["eps"])
    wq, wk = R.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    assert_bf16_close(q_out, wq, "q")
    assert_bf16_close(k_out, wk, "k")
    assert e_q.shape == (0, 32, 128) and e_k.shape == (0, 8, 128)


def test_in_place_on_strided_views_of_a_fused_projection():
    from tah_amd.kv_cache import qk_norm_rope
    c = make_case(21, 6, 4, 2)
    t = to_torch(c, "cpu")
    fused = torch.zeros(6, 4 + 2 + 2, 128, dtype=torch.bfloat16)
    fused[:, :4], fused[:, 4:6], fused[:, 6:] = t["q"], t["k"], t["v"]
    with emu_util.emulated():
        q_out, k_out = qk_norm_rope(fused[:, :4], fused[:, 4:6], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], in_place=True)
    wq, wk = R.qk_prep(c["q"], c["k"], c["qw"], c["kw"], c["cos"], c["sin"], c["eps"])
    assert q_out.data_ptr() == fused.data_ptr()
    assert_bf16_close(fused[:, :4], wq, "q")
    assert_bf16_close(fused[:, 4:6], wk, "k")
    assert torch.equal(fused[:, 6:], t["v"])


def test_fused_append_equals_norm_rope_then_append():
    from tah_amd.kv_cache import KvSlabs, qk_norm_rope
    c = make_case(22, 7, 4, 2)
    t = to_torch(c, "cpu")
    cu = torch.tensor([0, 3, 7], dtype=torch.int32)
    slot_of = torch.tensor([2, 0], dtype=torch.int32)
    with emu_util.emulated():
        a, b = KvSlabs(3, 5, 2, with_pos=True, device="cpu"), KvSlabs(3, 5, 2, with_pos=True, device="cpu")
        q1, none = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], v=t["v"], cache=a,
                                cu_new=cu, pos_new=t["pos"], slot_of=slot_of)
        q2, k2 = qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"])
        b.append(k2, t["v"], cu, pos_new=t["pos"], slot_of=slot_of)
        assert none is None and torch.equal(q1, q2)
        for x, y in ((a.k, b.k), (a.v, b.v), (a.pos, b.pos), (a.len, b.len), (a.overflow, b.overflow)):
            assert torch.equal(x, y)
        assert a.len.tolist() == [4, 0, 3]
        # a second append that does not fit: rows dropped, flag raised, as tah_kv_append does
        qk_norm_rope(t["q"][:3], t["k"][:3], t["qw"], t["kw"], t["cos"][:3], t["sin"][:3], c["eps"], v=t["v"][:3], cache=a,
                     cu_new=torch.tensor([0, 3], dtype=torch.int32), pos_new=t["pos"][:3], slot_of=torch.tensor([0], dtype=torch.int32))
        assert a.overflow.item() == 1 and a.len.tolist() == [5, 0, 3]


def test_argument_checks():
    from tah_amd import TahDuoError
    from tah_amd.kv_cache import qk_norm_rope
    c = make_case(23, 2, 2, 1)
    t = to_torch(c, "cpu")
    with emu_util.emulated():
        with pytest.raises(TahDuoError):
            qk_norm_rope(t["q"], t["k"], t["qw"].float(), t["kw"], t["cos"], t["sin"], 1e-6)
        with pytest.raises(TahDuoError):
            qk_norm_rope(t["q"], t["k"][:1], t["qw"], t["kw"], t["cos"], t["sin"], 1e-6)
        with pytest.raises(TahDuoError):
            qk_norm_rope(t["q"], t["k"], t["qw"], t["kw"], t["cos"][:, :64], t["sin"][:, :64], 1e-6)


@pytest.mark.parametrize("rows,hq,hkv,scale,n_partial", [(5, 4, 2, 1.0, None), (37, 2, 2, 20.0, 4), (3, 8, 1, 0.03, 8), (6, 32, 8, 1.0, 2)])
def test_backward_matches_analytic_gradients(rows, hq, hkv, scale, n_partial):
    from tests.qk_prep_cases import check_backward
    with emu_util.emulated():
        check_backward("cpu", 60 + rows, rows, hq, hkv, scale=scale, n_partial=n_partial)


def test_differentiable_form_refuses_what_it_cannot_differentiate():
    from tah_amd._capi import TahDuoError
    from tah_amd.kv_cache import qk_norm_rope
    c = make_case(70, 3, 2, 1)
    t = to_torch(c, "cpu")
    q = t["q"].clone().requires_grad_(True)
    with emu_util.emulated():
        with pytest.raises(TahDuoError, match="differentiable"):
            qk_norm_rope(q, t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], in_place=True)
        with pytest.raises(TahDuoError, match="differentiable"):
            qk_norm_rope(q, t["k"], t["qw"], t["kw"], t["cos"], t["sin"], c["eps"], norm_input=torch.zeros(3, 16, dtype=torch.bfloat16))
