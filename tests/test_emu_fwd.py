"""Runs the HIP forward and pack kernels on the CPU execution shim against the oracle.  No GPU."""
import numpy as np
import pytest
import torch

from oracle import duo_ref as R
from tests import emu_util
from tests.cases import add_score_drift, make_varlen_case, varlen_args

pytestmark = pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")

TOL = dict(atol=2e-2, rtol=2e-2)  # bf16 outputs vs float64-accumulated oracle on bf16-rounded inputs


def _to_dev(case):
    out = {}
    for k, v in case.items():
        if isinstance(v, np.ndarray):
            out[k] = torch.from_numpy(v.copy())
        elif torch.is_tensor(v):
            out[k] = v.to(torch.bfloat16)
        else:
            out[k] = v
    return out


def _oracle(dev):
    args = [a.float().numpy() if torch.is_tensor(a) and a.is_floating_point() else
            (a.numpy() if torch.is_tensor(a) else a) for a in varlen_args(dev)]
    return R.fwd(*args)


def _check(dev, got):
    o1, lse1, o2, lse2 = _oracle(dev)
    np.testing.assert_allclose(got[0].float().numpy(), o1, **TOL)
    np.testing.assert_allclose(got[1].numpy(), lse1, atol=2e-3, rtol=1e-3)
    np.testing.assert_allclose(got[2].float().numpy(), o2, **TOL)
    np.testing.assert_allclose(got[3].numpy(), lse2, atol=2e-3, rtol=1e-3)


@pytest.mark.parametrize("hq,hkv,seqlens,p", [
    (2, 1, [70], 0.3),           # G=2, one partial tile, depth-1 rows
    (2, 2, [130, 3], 0.1),       # G=1, 256-row tiles, second tiny sequence
    (4, 1, [65, 64], 0.2),       # G=4, 64-row tiles
    (2, 1, [3, 0, 9, 1] * 17 + [40], 0.3),   # 69 sequences: the tile lookup takes them 64 at a time
])
def test_fwd_kernel_on_cpu_shim(hq, hkv, seqlens, p):
    from tah_amd import ops
    dev = _to_dev(make_varlen_case(100 + hq, seqlens, p, Hq=hq, Hkv=hkv, D=128))
    with emu_util.emulated():
        got = ops.duo_fwd_varlen(*varlen_args(dev))
    _check(dev, got)


@pytest.mark.parametrize("nats_per_key", [0.25, 0.02])
def test_fwd_kernel_moving_softmax_reference(nats_per_key):
    """Scores that keep growing along the keys: per 64-key tile the row maximum rises by 16 nats (the
    exponent reference has to follow in every tile) or by 1.3 nats (it follows only every few tiles)."""
    from tah_amd import ops
    dev = _to_dev(add_score_drift(make_varlen_case(21, [200], 0.2, Hq=2, Hkv=1, D=128), nats_per_key))
    with emu_util.emulated():
        got = ops.duo_fwd_varlen(*varlen_args(dev))
    _check(dev, got)


def test_fwd_kernel_cache_prefix_and_strided_views():
    from tah_amd import ops
    dev = _to_dev(make_varlen_case(7, [5, 40], 0.5, Hq=2, Hkv=1, D=128, seqlens_k=[90, 40], extra_k2=70))
    # q/k/v as strided views of a fused [rows, Hq+2*Hkv, D] projection buffer
    fused = torch.zeros(dev["q1"].shape[0], 4, 128, dtype=torch.bfloat16)
    fused[:, :2] = dev["q1"]
    dev["q1"] = fused[:, :2]
    with emu_util.emulated():
        got = ops.duo_fwd_varlen(*varlen_args(dev))
    _check(dev, got)


def test_fwd_depth1_only_call():
    """Depth-1 queries alone against cached depth-0 and depth-1 keys (the per-layer call at depth 1)."""
    from tah_amd import ops
    dev = _to_dev(make_varlen_case(9, [33], 0.4, Hq=2, Hkv=1, D=128))
    want = _oracle(dev)
    d1 = dict(dev)
    d1["q1"] = dev["q1"][:0]
    d1["cu_q1"] = torch.zeros(2, dtype=torch.int32)
    with emu_util.emulated():
        got = ops.duo_fwd_varlen(*varlen_args(d1))
    assert got[0].shape[0] == 0
    np.testing.assert_allclose(got[2].float().numpy(), want[2], **TOL)


@pytest.mark.parametrize("B,S,p", [(3, 50, 0.3), (2, 9000, 0.06), (1, 1, 1.0), (4, 16, 0.0)])
def test_hard_index_bit_exact(B, S, p):
    from tah_amd import ops
    g = torch.Generator().manual_seed(B * 1000 + S)
    mask = torch.rand(B, S, generator=g) < p
    with emu_util.emulated():
        pos, flat, seq, cu = ops.hard_index_build(mask)
        n = int(cu[-1])
        pad = ops.pad_rows_build(cu, seq, n, max(int((cu[1:] - cu[:-1]).max()), 1))
    nz = mask.nonzero()
    assert cu.tolist() == [0] + torch.cumsum(mask.sum(1), 0).tolist()
    assert pos[:n].tolist() == nz[:, 1].tolist()
    assert seq[:n].tolist() == nz[:, 0].tolist()
    assert flat[:n].tolist() == (nz[:, 0] * S + nz[:, 1]).tolist()
    ridx, rcu = R.hard_index(mask.numpy())
    assert ridx.tolist() == pos[:n].tolist() and rcu.tolist() == cu.tolist()
    width = max(int(mask.sum(1).max()), 1)
    rank = torch.cat([torch.arange(int(c)) for c in mask.sum(1)]) if n else torch.zeros(0, dtype=torch.long)
    assert pad.tolist() == (nz[:, 0] * width + rank).tolist()


@pytest.mark.parametrize("dtype,inner", [(torch.bfloat16, (8,)), (torch.int64, ()), (torch.uint8, (3,)), (torch.float32, (5, 2))])
def test_rows_copy_bit_exact(dtype, inner):
    from tah_amd import ops
    g = torch.Generator().manual_seed(3)
    src = torch.randint(0, 100, (40,) + inner, generator=g).to(dtype)
    rows = torch.randperm(40, generator=g)[:17].to(torch.int32)
    with emu_util.emulated():
        out = torch.zeros((17,) + inner, dtype=dtype)
        ops.rows_copy(src, rows, out, None, 17)
        back = torch.full_like(src, 7)
        ops.rows_copy(out, None, back, rows, 17)
    assert torch.equal(out, src[rows.long()])
    want = torch.full_like(src, 7)
    want[rows.long()] = src[rows.long()]
    assert torch.equal(back, want)
