"""Golden fixtures (tests/golden/*.npz): the oracle must reproduce them (CPU), and the HIP path must match them
on the GPU through the C ABI (and, without a GPU, on the CPU execution shim)."""
import os

import numpy as np
import pytest
import torch

from oracle import duo_oracle as O
from oracle import duo_ref as R
from tests import emu_util
from tests.cases import VARLEN_KEYS, build_slabs

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def load_prefill():
    z = np.load(os.path.join(G, "prefill_small.npz"))
    c = {k: (_bf16(z[k]) if k in ("q1", "k1", "v1", "q2", "k2", "v2") else z[k]) for k in VARLEN_KEYS if k != "scale"}
    c["scale"] = float(z["scale"])
    return z, c


def test_oracle_reproduces_prefill_fixture():
    z, c = load_prefill()
    args = [c[k].float().numpy() if torch.is_tensor(c[k]) else c[k] for k in VARLEN_KEYS]
    for name, got in zip(("o1", "lse1", "o2", "lse2"), R.fwd(*args)):
        np.testing.assert_allclose(got, z[name], atol=1e-6, rtol=1e-5)
    for name, got in zip(("o1", "lse1", "o2", "lse2"), O.duo_rows_f64(*args)):
        np.testing.assert_allclose(got, z[name], atol=3e-6, rtol=1e-5)
    grads = R.bwd(*args, _bf16(z["do1"]).float().numpy(), _bf16(z["do2"]).float().numpy())
    for n, g in zip(("dq1", "dk1", "dv1", "dq2", "dk2", "dv2"), grads):
        np.testing.assert_allclose(g, z[n], atol=1e-6, rtol=1e-5)


def test_oracle_reproduces_pack_fixture():
    z = np.load(os.path.join(G, "pack_small.npz"))
    mask, x = torch.from_numpy(z["mask"]), torch.from_numpy(z["x"])
    idx, cu = O.hard_index(mask)
    assert idx.tolist() == z["idx"].tolist() and cu.tolist() == z["cu"].tolist()
    pad, gx = O.gather_active(mask, x)
    assert np.array_equal(pad.numpy(), z["pad_mask"]) and np.array_equal(gx.numpy(), z["gathered"])


def _check_prefill(dev_of):
    from tah_amd import ops
    z, c = load_prefill()
    d = {k: (dev_of(v) if torch.is_tensor(v) else (dev_of(torch.from_numpy(v)) if isinstance(v, np.ndarray) else v))
         for k, v in c.items()}
    o1, lse1, o2, lse2 = ops.duo_fwd_varlen(*[d[k] for k in VARLEN_KEYS])
    np.testing.assert_allclose(o1.float().cpu().numpy(), z["o1"], atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(o2.float().cpu().numpy(), z["o2"], atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(lse1.cpu().numpy(), z["lse1"], atol=5e-3, rtol=1e-3)
    np.testing.assert_allclose(lse2.cpu().numpy(), z["lse2"], atol=5e-3, rtol=1e-3)
    do1, do2 = dev_of(_bf16(z["do1"])), dev_of(_bf16(z["do2"]))
    grads = ops.duo_bwd_varlen(d["q1"], d["k1"], d["v1"], o1, lse1, do1, d["cu_q1"], d["cu_k1"], d["q2"], d["k2"], d["v2"],
                               o2, lse2, do2, d["pos_q2"], d["pos_k2"], d["cu_q2"], d["cu_k2"], d["scale"])
    for n, g in zip(("dq1", "dk1", "dv1", "dq2", "dk2", "dv2"), grads):
        err = np.abs(g.float().cpu().numpy() - z[n]).max() / np.abs(z[n]).max()
        assert err <= 2e-2, (n, err)


def _check_decode(device):
    from tah_amd import kv_cache
    z = np.load(os.path.join(G, "decode_small.npz"))
    c = {k: _bf16(z[k]) for k in ("q1", "k1", "v1", "q2", "k2", "v2")}
    c.update(cu_k1=z["cu_k1"], cu_k2=z["cu_k2"], pos_k2=z["pos_k2"], lens=z["lens"].tolist())
    s1, s2 = build_slabs(c, 256, 64, device=device)
    slot = torch.arange(3, dtype=torch.int32, device=device)
    qpos = torch.from_numpy(z["q_pos"]).to(device)
    hr = torch.from_numpy(z["hard_rows"]).to(device)
    o0, l0 = kv_cache.decode(c["q1"].to(device), slot, qpos, s1, None, scale=float(z["scale"]), depth=0, return_lse=True)
    o1, l1 = kv_cache.decode(c["q2"].to(device), hr, qpos[hr.long()], s1, s2, scale=float(z["scale"]), depth=1, return_lse=True)
    np.testing.assert_allclose(o0.float().cpu().numpy(), z["o_depth0"], atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(o1.float().cpu().numpy(), z["o_depth1"], atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(l0.cpu().numpy(), z["lse_depth0"], atol=5e-3, rtol=1e-3)
    np.testing.assert_allclose(l1.cpu().numpy(), z["lse_depth1"], atol=5e-3, rtol=1e-3)


def _check_pack(device):
    from tah_amd.pack import HardIndex, gather_active, scatter_back
    z = np.load(os.path.join(G, "pack_small.npz"))
    mask, x = torch.from_numpy(z["mask"]).to(device), torch.from_numpy(z["x"]).to(device)
    idx = HardIndex(mask)
    assert idx.pos.cpu().tolist() == z["idx"].tolist() and idx.cu.cpu().tolist() == z["cu"].tolist()
    pad, gx = gather_active(mask, x)
    assert np.array_equal(pad.cpu().numpy(), z["pad_mask"]) and np.array_equal(gx.cpu().numpy(), z["gathered"])
    dest = torch.full_like(x, -7)
    assert np.array_equal(scatter_back(mask, gx, dest).cpu().numpy(), z["scattered"])
    am = torch.from_numpy(z["assignment_mask"]).to(device)
    assert np.array_equal(scatter_back(mask, gx, dest, assignment_mask=am).cpu().numpy(), z["scattered_assigned"])


def _load_qk_prep():
    z = np.load(os.path.join(G, "qk_prep_small.npz"))
    return z, {k: _bf16(z[k]) for k in ("q", "k", "v", "qw", "kw", "cos", "sin", "q_out", "k_out")}


def test_oracle_reproduces_qk_prep_fixture():
    """The fixture's expected values come from the third-party modules themselves."""
    from oracle import qk_prep_ref as Q
    from tests.qk_prep_cases import assert_bf16_close
    z, c = _load_qk_prep()
    f = lambda k: c[k].float().numpy()
    gq, gk = Q.qk_prep(f("q"), f("k"), f("qw"), f("kw"), f("cos"), f("sin"), float(z["eps"]))
    assert np.mean(gq == f("q_out")) > 0.999 and np.mean(gk == f("k_out")) > 0.999
    assert_bf16_close(torch.from_numpy(gq), f("q_out"), "q")
    assert_bf16_close(torch.from_numpy(gk), f("k_out"), "k")


def _check_qk_prep(device):
    from tah_amd.kv_cache import qk_norm_rope
    from tests.qk_prep_cases import assert_bf16_close
    z, c = _load_qk_prep()
    d = {k: v.to(device) for k, v in c.items()}
    q_out, k_out = qk_norm_rope(d["q"], d["k"], d["qw"], d["kw"], d["cos"], d["sin"], float(z["eps"]))
    assert_bf16_close(q_out, c["q_out"].float().numpy(), "q vs fixture")
    assert_bf16_close(k_out, c["k_out"].float().numpy(), "k vs fixture")


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_kernels_on_cpu_shim_match_fixtures():
    with emu_util.emulated():
        _check_prefill(lambda t: t)
        _check_decode("cpu")
        _check_pack("cpu")
        _check_qk_prep("cpu")


@pytest.mark.gpu
def test_hip_path_matches_fixtures():
    _check_prefill(lambda t: t.cuda())
    _check_decode("cuda")
    _check_pack("cuda")
    _check_qk_prep("cuda")
