"""Backward kernels (delta, dQ, dK/dV) on the CPU execution shim against the analytic C oracle.  No GPU."""
import numpy as np
import pytest
import torch

from oracle import duo_ref as R
from tests import emu_util
from tests.cases import make_varlen_case, varlen_args
from tests.test_emu_fwd import _to_dev

pytestmark = pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")

NAMES = ("dq1", "dk1", "dv1", "dq2", "dk2", "dv2")


def run_bwd(dev, seed, schedule=None, ds_workspace=None, want_oracle=True, **bwd_kw):
    """Forward + backward through tah_amd.ops; returns kernel grads and oracle grads (on the bf16-rounded inputs;
    None when a launch-order table is given: that call is only compared with the one without).
    ``ds_workspace=False``: the three-kernel backward; None: the package's default (dS exchange where it applies)."""
    from tah_amd import ops
    g = torch.Generator().manual_seed(seed)
    mk = lambda t: torch.randn(t.shape, generator=g).to(torch.bfloat16).to(t.device)
    do1, do2 = mk(dev["q1"]), mk(dev["q2"])
    o1, lse1, o2, lse2 = ops.duo_fwd_varlen(*varlen_args(dev), schedule=schedule)
    got = ops.duo_bwd_varlen(dev["q1"], dev["k1"], dev["v1"], o1, lse1, do1, dev["cu_q1"], dev["cu_k1"],
                             dev["q2"], dev["k2"], dev["v2"], o2, lse2, do2, dev["pos_q2"], dev["pos_k2"],
                             dev["cu_q2"], dev["cu_k2"], dev["scale"], schedule=schedule, ds_workspace=ds_workspace, **bwd_kw)
    if schedule is not None or not want_oracle:
        return got, None
    host = [a.float().cpu().numpy() if torch.is_tensor(a) and a.is_floating_point() else
            (a.cpu().numpy() if torch.is_tensor(a) else a) for a in varlen_args(dev)]
    want = R.bwd(*host, do1.float().cpu().numpy(), do2.float().cpu().numpy())
    return got, want


def check_grads(got, want, max_rel=2e-2, mean_rel=1e-2):
    """max|a-b| <= max_rel * max|b| and mean|a-b| <= mean_rel * mean|b| per gradient tensor (bf16 outputs);
    a gradient that is identically ~0 in the reference (single visible key) is held to 1e-3 absolute."""
    out = {}
    for n, a, b in zip(NAMES, got, want):
        if b.size == 0:
            continue
        d = np.abs(a.float().cpu().numpy().astype(np.float64) - b)
        if np.abs(b).max() < 1e-3:
            assert d.max() <= 1e-3, f"{n}: reference is ~0, max-abs-err {d.max():.3e}"
            out[n] = (float(d.max()), 0.0)
            continue
        ma, mr = d.max() / np.abs(b).max(), d.mean() / np.abs(b).mean()
        out[n] = (float(ma), float(mr))
        assert ma <= max_rel and mr <= mean_rel, f"{n}: max-err/max|ref| {ma:.3e} (tol {max_rel}), mean-rel-err {mr:.3e} (tol {mean_rel})"
    return out


@pytest.mark.parametrize("hq,hkv,seqlens,p,kw", [
    (2, 1, [70], 0.3, {}),
    (2, 2, [130, 3], 0.1, {}),
    (4, 1, [65, 64], 0.2, {}),
    (2, 1, [5, 40], 0.5, dict(seqlens_k=[90, 40], extra_k2=70)),
])
def test_bwd_kernels_on_cpu_shim(hq, hkv, seqlens, p, kw):
    dev = _to_dev(make_varlen_case(200 + hq, seqlens, p, Hq=hq, Hkv=hkv, D=128, **kw))
    with emu_util.emulated():
        got, want = run_bwd(dev, 5)
    print(check_grads(got, want))


@pytest.mark.parametrize("hq,hkv,seqlens,p,kw", [
    (2, 1, [70, 130], 0.3, {}),
    (1, 1, [300], 0.2, {}),
    (4, 1, [5, 40], 0.5, dict(seqlens_k=[90, 40], extra_k2=70)),
])
def test_ds_exchange_against_three_kernel_backward_on_cpu_shim(hq, hkv, seqlens, p, kw):
    """The backward that hands dS from the dK/dV kernel to the dQ product through a workspace: dK and dV are the
    three-kernel path's to the bit, dQ meets the oracle; a workspace sized with the per-sequence bounds gives
    the same bits as one sized from the totals, and a workspace that is too small is refused."""
    from tah_amd import ops
    from tah_amd._capi import TahDuoError
    dev = _to_dev(make_varlen_case(300 + hq, seqlens, p, Hq=hq, Hkv=hkv, D=128, **kw))
    with emu_util.emulated():
        old, want = run_bwd(dev, 6, ds_workspace=False)
        new, _ = run_bwd(dev, 6, want_oracle=False)
        mk1 = int(np.diff(dev["cu_k1"].cpu().numpy()).max())
        mk2 = int(np.diff(dev["cu_k2"].cpu().numpy()).max()) if dev["k2"].shape[0] else 0
        need = ops.duo_bwd_workspace_bytes(len(seqlens), hq, hkv, dev["q1"].shape[0], dev["k1"].shape[0], dev["q2"].shape[0],
                                           dev["k2"].shape[0], mk1, mk2)
        assert 0 < need <= ops.duo_bwd_workspace_bytes(len(seqlens), hq, hkv, dev["q1"].shape[0], dev["k1"].shape[0],
                                                       dev["q2"].shape[0], dev["k2"].shape[0])
        ws = torch.full((need,), 0xFF, dtype=torch.uint8)  # NaN patterns: a block read without having been written shows
        tight, _ = run_bwd(dev, 6, ds_workspace=ws, want_oracle=False, max_seqlen_k1=mk1, max_seqlen_k2=mk2)
        with pytest.raises(TahDuoError):
            run_bwd(dev, 6, ds_workspace=ws[: need - 16], want_oracle=False, max_seqlen_k1=mk1, max_seqlen_k2=mk2)
    print(check_grads(new, want))
    for i, n in enumerate(NAMES):
        assert torch.equal(new[i], tight[i]), n
        if n[1] != "q":
            assert torch.equal(new[i], old[i]), n
    assert any(not torch.equal(new[i], old[i]) for i in (0, 3)) or dev["q1"].shape[0] < 8
