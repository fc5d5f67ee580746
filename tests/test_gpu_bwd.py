"""GPU parity: backward kernels through the C ABI vs the analytic C oracle / torch fp32 autograd."""
import numpy as np
import pytest
import torch

from oracle import duo_oracle as O
from tests.cases import make_varlen_case, varlen_args
from tests.gpu_util import to_device
from tests.test_emu_bwd import NAMES, check_grads, run_bwd

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("hq,hkv,seqlens,p,seed,kw", [
    (16, 8, [512], 0.06, 1235, {}),
    (16, 8, [300, 1000, 17, 129], 0.10, 2, {}),
    (8, 8, [257, 64], 0.2, 3, {}),
    (16, 4, [700], 0.3, 4, {}),
    (8, 1, [130, 31], 0.5, 5, {}),
    (16, 8, [1], 1.0, 6, {}),
    (16, 8, [777], 0.0, 7, {}),
    (16, 8, [640], 1.0, 8, {}),
    (16, 8, [40, 1, 300], 0.3, 11, dict(seqlens_k=[500, 900, 300], extra_k2=100)),
])
def test_bwd_matches_oracle(hq, hkv, seqlens, p, seed, kw):
    print(f"bwd case hq={hq} hkv={hkv} seqlens={seqlens} p={p} seed={seed} {kw}", flush=True)
    dev = to_device(make_varlen_case(seed, seqlens, p, Hq=hq, Hkv=hkv, D=128, **kw))
    got, want = run_bwd(dev, seed + 100)
    torch.cuda.synchronize()
    print(check_grads(got, want), flush=True)


@pytest.mark.parametrize("ds_workspace", [None, False], ids=["ds-exchange", "three-kernel"])
def test_bwd_is_deterministic(ds_workspace):
    dev = to_device(make_varlen_case(21, [900, 200], 0.1))
    a, _ = run_bwd(dev, 1, ds_workspace=ds_workspace, want_oracle=False)
    b, _ = run_bwd(dev, 1, ds_workspace=ds_workspace, want_oracle=False)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


@pytest.mark.parametrize("hq,hkv,seqlens,p,seed,kw", [
    (16, 8, [300, 1000, 17, 129], 0.10, 2, {}),
    (8, 8, [257, 64], 0.2, 3, {}),
    (16, 4, [700], 0.3, 4, {}),
    (16, 8, [40, 1, 300], 0.3, 11, dict(seqlens_k=[500, 900, 300], extra_k2=100)),
    (16, 8, [2500], 0.06, 12, {}),
])
def test_ds_exchange_against_three_kernel_backward(hq, hkv, seqlens, p, seed, kw):
    """Both backward paths on the same inputs: dK / dV equal to the bit (same kernel arithmetic), dQ of both within
    the tolerance of the oracle; the exchange path with a caller's workspace sized by the per-sequence bounds and
    pre-filled with NaN patterns (a block read before it was written would show) gives the default path's bits."""
    from tah_amd import ops
    print(f"ds exchange case hq={hq} hkv={hkv} seqlens={seqlens} p={p} seed={seed} {kw}", flush=True)
    dev = to_device(make_varlen_case(seed, seqlens, p, Hq=hq, Hkv=hkv, D=128, **kw))
    old, want = run_bwd(dev, seed + 100, ds_workspace=False)
    new, _ = run_bwd(dev, seed + 100, want_oracle=False)
    mk1 = int(np.diff(dev["cu_k1"].cpu().numpy()).max())
    mk2 = int(np.diff(dev["cu_k2"].cpu().numpy()).max()) if dev["k2"].shape[0] else 0
    need = ops.duo_bwd_workspace_bytes(len(seqlens), hq, hkv, dev["q1"].shape[0], dev["k1"].shape[0], dev["q2"].shape[0],
                                       dev["k2"].shape[0], mk1, mk2)
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")
    tight, _ = run_bwd(dev, seed + 100, ds_workspace=ws, want_oracle=False, max_seqlen_k1=mk1, max_seqlen_k2=mk2)
    torch.cuda.synchronize()
    print(check_grads(new, want), flush=True)
    for i, n in enumerate(NAMES):
        assert torch.equal(new[i], tight[i]), n
        if n[1] != "q":
            assert torch.equal(new[i], old[i]), n


def test_bwd_full_size_training_config_vs_torch_fp32():
    """BASELINE config 3: 8192 packed tokens in 4 documents, p=0.10, dO ~ N(0,1); torch fp32 autograd on the GPU
    through the dense-mask formulation is the reference at this size."""
    from tah_amd import ops
    g = torch.Generator().manual_seed(1237)
    cuts = sorted((torch.randperm(8192 - 4 * 256, generator=g)[:3]).tolist())
    lens = [b - a + 256 for a, b in zip([0] + cuts, cuts + [8192 - 4 * 256])]
    assert sum(lens) == 8192 and min(lens) >= 256
    print("doc lengths", lens, flush=True)
    dev = to_device(make_varlen_case(1237, lens, 0.10))
    gen = torch.Generator().manual_seed(5)
    do1 = torch.randn(dev["q1"].shape, generator=gen).to(torch.bfloat16).cuda()
    do2 = torch.randn(dev["q2"].shape, generator=gen).to(torch.bfloat16).cuda()
    o1, lse1, o2, lse2 = ops.duo_fwd_varlen(*varlen_args(dev))
    got = ops.duo_bwd_varlen(dev["q1"], dev["k1"], dev["v1"], o1, lse1, do1, dev["cu_q1"], dev["cu_k1"],
                             dev["q2"], dev["k2"], dev["v2"], o2, lse2, do2, dev["pos_q2"], dev["pos_k2"],
                             dev["cu_q2"], dev["cu_k2"], dev["scale"])
    torch.cuda.synchronize()
    leaf = {k: (v.float().requires_grad_(True) if torch.is_tensor(v) and v.is_floating_point() else
                (v.cpu().numpy() if torch.is_tensor(v) else v)) for k, v in dev.items()}
    torch_default = torch.get_default_device()
    torch.set_default_device("cuda")
    try:
        r1, r2 = O.duo_varlen_torch(*varlen_args(leaf))
    finally:
        torch.set_default_device(torch_default)
    ((r1 * do1.float()).sum() + (r2 * do2.float()).sum()).backward()
    want = [leaf[n].grad.cpu().numpy() for n in ("q1", "k1", "v1", "q2", "k2", "v2")]
    print("full-size fwd+bwd:", check_grads(got, want), flush=True)


def test_fwd_bwd_headline_seq8192_vs_torch_fp32():
    """The headline shape (one sequence of 8192 tokens, 6 % hard, Hq=16, Hkv=8, D=128): outputs of both depths and
    all six gradients against torch fp32 autograd through the dense-mask formulation on the device."""
    from tah_amd import ops
    from tests.gpu_util import assert_close
    dev = to_device(make_varlen_case(1238, [8192], 0.06, std=0.5))
    gen = torch.Generator().manual_seed(6)
    do1 = torch.randn(dev["q1"].shape, generator=gen).to(torch.bfloat16).cuda()
    do2 = torch.randn(dev["q2"].shape, generator=gen).to(torch.bfloat16).cuda()
    o1, lse1, o2, lse2 = ops.duo_fwd_varlen(*varlen_args(dev))
    got = ops.duo_bwd_varlen(dev["q1"], dev["k1"], dev["v1"], o1, lse1, do1, dev["cu_q1"], dev["cu_k1"],
                             dev["q2"], dev["k2"], dev["v2"], o2, lse2, do2, dev["pos_q2"], dev["pos_k2"],
                             dev["cu_q2"], dev["cu_k2"], dev["scale"])
    torch.cuda.synchronize()
    leaf = {k: (v.float().requires_grad_(True) if torch.is_tensor(v) and v.is_floating_point() else
                (v.cpu().numpy() if torch.is_tensor(v) else v)) for k, v in dev.items()}
    torch_default = torch.get_default_device()
    torch.set_default_device("cuda")
    try:
        r1, r2 = O.duo_varlen_torch(*varlen_args(leaf))
    finally:
        torch.set_default_device(torch_default)
    print("headline fwd: o1", assert_close(o1, r1.detach().cpu().numpy(), "headline o1"),
          "o2", assert_close(o2, r2.detach().cpu().numpy(), "headline o2"), flush=True)
    ((r1 * do1.float()).sum() + (r2 * do2.float()).sum()).backward()
    want = [leaf[n].grad.cpu().numpy() for n in ("q1", "k1", "v1", "q2", "k2", "v2")]
    print("headline fwd+bwd:", check_grads(got, want), flush=True)
