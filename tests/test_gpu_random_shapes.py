"""GPU parity on seeded random shapes: forward and backward through the C ABI vs the CPU oracle, over
group sizes, ragged batches, cached prefixes, extra depth-1 keys and hard fractions drawn at random."""
import numpy as np
import pytest
import torch

from tests.cases import make_varlen_case, varlen_args
from tests.gpu_util import assert_close, oracle_fwd, to_device
from tests.test_emu_bwd import check_grads, run_bwd

pytestmark = pytest.mark.gpu


def _draw(seed):
    g = np.random.default_rng(seed)
    hkv = int(g.choice([1, 2, 4, 8]))
    hq = hkv * int(g.choice([1, 2, 4, 8]))
    while hq > 32:
        hq //= 2
    nseq = int(g.integers(1, 6))
    seqlens = [int(x) for x in np.maximum(1, (g.pareto(1.5, nseq) * 120).astype(int) % 900)]
    p = float(g.choice([0.0, 0.03, 0.1, 0.3, 0.7, 1.0]))
    kw = {}
    if g.random() < 0.4:  # cached prefix: more keys than queries, some earlier depth-1 rows
        kw = dict(seqlens_k=[n + int(g.integers(0, 300)) for n in seqlens], extra_k2=int(g.integers(0, 80)))
    return hq, hkv, seqlens, p, kw


@pytest.mark.parametrize("seed", list(range(500, 524)))
def test_random_shape_forward_and_backward(seed):
    hq, hkv, seqlens, p, kw = _draw(seed)
    print(f"case random seed={seed} hq={hq} hkv={hkv} seqlens={seqlens} p={p} {kw}", flush=True)
    from tah_amd import ops
    dev = to_device(make_varlen_case(seed, seqlens, p, Hq=hq, Hkv=hkv, D=128, **kw))
    out = ops.duo_fwd_varlen(*varlen_args(dev))
    torch.cuda.synchronize()
    o1, lse1, o2, lse2 = oracle_fwd(dev)
    assert_close(out[0], o1, "o1")
    assert_close(out[2], o2, "o2")
    np.testing.assert_allclose(out[1].cpu().numpy(), lse1, atol=5e-3, rtol=1e-3)
    np.testing.assert_allclose(out[3].cpu().numpy(), lse2, atol=5e-3, rtol=1e-3)
    got, want = run_bwd(dev, seed + 1)
    torch.cuda.synchronize()
    check_grads(got, want)
    # the same calls with the launch-order table of the batch: bit-identical outputs and gradients
    sched = ops.duo_schedule(dev["cu_q1"], dev["cu_k1"], dev["cu_q2"], dev["cu_k2"], dev["pos_q2"], hq, hkv,
                             dev["q1"].shape[0], dev["k1"].shape[0], dev["k2"].shape[0])
    assert (sched is None) == (len(seqlens) == 1)
    if sched is not None:
        for a, b in zip(out, ops.duo_fwd_varlen(*varlen_args(dev), schedule=sched)):
            assert torch.equal(a, b)
        got2, _ = run_bwd(dev, seed + 1, schedule=sched)
        for a, b in zip(got, got2):
            assert torch.equal(a, b)


@pytest.mark.parametrize("hq,hkv,seqlens,p", [
    (4, 2, [32] * 150 + [0] * 3 + [100] * 20, 0.2),        # 173 sequences: the tile lookup takes them 64 at a time
    (2, 1, [1, 7, 0, 130] * 40 + [500], 0.3),              # 161 ragged ones, empty ones among them
])
def test_many_short_sequences_forward_and_backward(hq, hkv, seqlens, p):
    from tah_amd import ops
    dev = to_device(make_varlen_case(77, seqlens, p, Hq=hq, Hkv=hkv, D=128))
    out = ops.duo_fwd_varlen(*varlen_args(dev))
    o1, lse1, o2, lse2 = oracle_fwd(dev)
    assert_close(out[0], o1, "o1")
    assert_close(out[2], o2, "o2")
    np.testing.assert_allclose(out[1].cpu().numpy(), lse1, atol=5e-3, rtol=1e-3)
    got, want = run_bwd(dev, 78)
    check_grads(got, want)
    sched = ops.duo_schedule(dev["cu_q1"], dev["cu_k1"], dev["cu_q2"], dev["cu_k2"], dev["pos_q2"], hq, hkv,
                             dev["q1"].shape[0], dev["k1"].shape[0], dev["k2"].shape[0])
    for a, b in zip(out, ops.duo_fwd_varlen(*varlen_args(dev), schedule=sched)):
        assert torch.equal(a, b)
    got2, _ = run_bwd(dev, 78, schedule=sched)
    for a, b in zip(got, got2):
        assert torch.equal(a, b)


def _draw_decode(seed):
    g = np.random.default_rng(seed)
    hkv = int(g.choice([1, 2, 4, 8]))
    hq = min(32, hkv * int(g.choice([1, 2, 4, 8])))
    nseq = int(g.integers(1, 9))
    lens = [int(x) for x in 1 + (g.pareto(1.2, nseq) * 300).astype(int) % 5000]
    return hq, hkv, lens, float(g.choice([0.0, 0.06, 0.3, 1.0])), bool(g.random() < 0.5)


@pytest.mark.parametrize("seed", list(range(600, 616)))
def test_random_shape_decode(seed):
    from tests.cases import make_decode_case
    from tests.test_gpu_decode import oracle_decode_c, run_decode
    hq, hkv, lens, p, fused = _draw_decode(seed)
    print(f"case random decode seed={seed} hq={hq} hkv={hkv} lens={lens} p={p} fused={fused}", flush=True)
    c = make_decode_case(seed, lens, p, Hq=hq, Hkv=hkv)
    got = run_decode(c, 5120, 5120, fused)
    w0, wl0, w1, wl1 = oracle_decode_c(c)
    assert_close(got[0], w0, "decode o depth0")
    np.testing.assert_allclose(got[1].cpu().numpy(), wl0, atol=5e-3, rtol=1e-3)
    if len(c["hard_rows"]):
        assert_close(got[2], w1, "decode o depth1")
        np.testing.assert_allclose(got[3].cpu().numpy(), wl1, atol=5e-3, rtol=1e-3)
