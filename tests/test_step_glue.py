"""Glue kernels of a generation step (tah_step_begin, tah_decider_tail) against the torch operations they replace.
step_begin is gathers and selects: exact.  decider_tail follows the eager bf16 arithmetic (`h @ w2.T + b2` in bf16,
sigmoid in float32); its float32 dot product runs in another order than the library GEMM's, so a row whose probability
sits within a bf16 step of the threshold could decide differently: the test's thresholds keep clear of the rows."""
import pytest
import torch

from tests import emu_util

BF = torch.bfloat16


def _step_begin_case(dev, B=5, H=96, V=50, L=40, packed=True):
    from tah_amd import ops
    from tests.test_linear_rows import unpack_rows
    g = torch.Generator().manual_seed(3)
    embed = torch.randn(V, H, generator=g).to(BF).to(dev)
    cos_t, sin_t = torch.randn(L, 128, generator=g).to(BF).to(dev), torch.randn(L, 128, generator=g).to(BF).to(dev)
    tok = torch.randint(0, V, (B,), generator=g).to(dev)
    pos = torch.randint(0, L + 5, (B,), generator=g).to(torch.int32).to(dev)   # some past the tables: clamped
    fin = (torch.rand(B, generator=g) < 0.4).to(dev)
    x = torch.full((B, H), 9.0, dtype=BF, device=dev)
    xp = torch.zeros(32 * H, dtype=BF, device=dev) if packed else None
    cr, sr = torch.empty(B, 128, dtype=BF, device=dev), torch.empty(B, 128, dtype=BF, device=dev)
    slot, qpos = torch.empty(B, dtype=torch.int32, device=dev), torch.empty(B, dtype=torch.int32, device=dev)
    act = torch.empty(B, dtype=torch.bool, device=dev)
    ops.step_begin(tok, pos, fin, embed, cos_t, sin_t, x=x, x_packed=xp, cos_rows=cr, sin_rows=sr, slot=slot, q_pos=qpos, active=act)
    at = pos.long().clamp(0, L - 1)
    rows = torch.arange(B, dtype=torch.int32, device=dev)
    assert torch.equal(act, ~fin)
    assert torch.equal(slot, torch.where(~fin, rows, torch.full_like(rows, -1)))
    assert torch.equal(qpos, torch.where(~fin, pos, torch.full_like(pos, -1)))
    assert torch.equal(cr, cos_t[at]) and torch.equal(sr, sin_t[at])
    assert torch.equal(x, embed[tok])
    if packed:
        full = unpack_rows(xp.cpu(), H)
        assert torch.equal(full[:B], x.cpu()) and not full[B:].any()


def _decider_tail_case(dev, B=9, W=64):
    from tah_amd import ops
    g = torch.Generator().manual_seed(5)
    h = torch.relu(torch.randn(B, W, generator=g)).to(BF).to(dev)
    w2 = (torch.randn(1, W, generator=g) * 0.3).to(BF).to(dev)
    b2 = torch.tensor([0.25], dtype=BF, device=dev)
    pos = torch.randint(0, 100, (B,), generator=g).to(torch.int32).to(dev)
    act = (torch.rand(B, generator=g) < 0.8).to(dev)
    prob = torch.sigmoid((h.double() @ w2.double().t()).to(BF).add(b2).float()).view(-1)   # exact sums, eager roundings
    srt = prob.sort().values
    thr = float((srt[B // 2 - 1] + srt[B // 2]) / 2)   # half of the rows above, the threshold between two of them
    hard = torch.empty(B, dtype=torch.bool, device=dev)
    hi, slot, qp = (torch.empty(B, dtype=torch.int32, device=dev) for _ in range(3))
    ops.decider_tail(h, w2.reshape(-1), b2, thr, hard=hard, active=act, pos=pos, hard_i32=hi, slot=slot, q_pos=qp)
    want = (prob > thr) & act
    assert want.any() and not want.all()
    rows = torch.arange(B, dtype=torch.int32, device=dev)
    assert torch.equal(hard, want) and torch.equal(hi, want.to(torch.int32))
    assert torch.equal(slot, torch.where(want, rows, torch.full_like(rows, -1)))
    assert torch.equal(qp, torch.where(want, pos, torch.full_like(pos, -1)))
    # everything optional left out: only the decision, for all rows
    ops.decider_tail(h, w2.reshape(-1), None, thr, hard=hard)
    assert torch.equal(hard, torch.sigmoid((h.double() @ w2.double().t()).to(BF).float()).view(-1) > thr)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_step_glue_on_cpu_shim():
    with emu_util.emulated():
        _step_begin_case("cpu")
        _step_begin_case("cpu", B=33, H=72, packed=False)   # more than 32 rows: no packed form
        _decider_tail_case("cpu")


@pytest.mark.gpu
def test_step_glue_gpu():
    _step_begin_case("cuda", B=32, H=2048, V=5000, L=1600)
    _step_begin_case("cuda", B=40, H=1000, V=777, L=64, packed=False)
    _decider_tail_case("cuda", B=32, W=512)
    _decider_tail_case("cuda", B=7, W=2048)
