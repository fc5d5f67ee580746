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


def _step_begin_phase_case(dev, B=6, H=64, V=30, L=50):
    """Rows at their second latent iteration take their input from x_alt and append at the depth-1 row count."""
    from tah_amd import ops
    g = torch.Generator().manual_seed(4)
    embed = torch.randn(V, H, generator=g).to(BF).to(dev)
    alt = torch.randn(B, H, generator=g).to(BF).to(dev)
    cos_t, sin_t = torch.randn(L, 128, generator=g).to(BF).to(dev), torch.randn(L, 128, generator=g).to(BF).to(dev)
    tok = torch.randint(0, V, (B,), generator=g).to(dev)
    pos = torch.randint(0, L, (B,), generator=g).to(torch.int32).to(dev)
    hlen = torch.randint(0, 9, (B,), generator=g).to(torch.int32).to(dev)
    fin = torch.tensor([False, True, False, False, True, False]).to(dev)
    phase = torch.tensor([1, 1, 0, 0, 0, 1], dtype=torch.int32).to(dev)
    x = torch.empty(B, H, dtype=BF, device=dev)
    xp = torch.zeros(32 * H, dtype=BF, device=dev)
    cr, sr = torch.empty(B, 128, dtype=BF, device=dev), torch.empty(B, 128, dtype=BF, device=dev)
    slot, qpos, qd, at = (torch.empty(B, dtype=torch.int32, device=dev) for _ in range(4))
    act, el = torch.empty(B, dtype=torch.bool, device=dev), torch.empty(B, dtype=torch.bool, device=dev)
    ops.step_begin(tok, pos, fin, embed, cos_t, sin_t, x=x, x_packed=xp, cos_rows=cr, sin_rows=sr, slot=slot, q_pos=qpos, active=act,
                   phase=phase, x_alt=alt, hard_len=hlen, q_depth=qd, append_at=at, eligible=el)
    second = phase != 0
    assert torch.equal(x, torch.where(second[:, None], alt, embed[tok]))
    assert torch.equal(qd, phase) and torch.equal(at, torch.where(second, hlen, pos))
    assert torch.equal(act, ~fin) and torch.equal(el, ~fin & ~second)


def _greedy_tick_case(dev, B=7, V=304, limit=5, eos=11):
    """Every combination of finished / phase / hard_now, a row reaching the limit and a row hitting end-of-sequence."""
    from tah_amd import ops
    g = torch.Generator().manual_seed(6)
    cur = torch.randn(B, V, generator=g).to(BF)
    prev = torch.randn(B, V, generator=g).to(BF)
    cur[5, eos] = 50.0                          # row 5 chooses the end-of-sequence token
    fin = torch.tensor([False, True, False, False, False, False, False])
    phase = torch.tensor([0, 0, 0, 1, 1, 0, 0], dtype=torch.int32)
    hard = torch.tensor([True, True, False, False, True, False, False])      # (ignored at phase 1)
    out_len = torch.tensor([1, 2, 3, 1, 2, 2, limit - 1], dtype=torch.int32)  # row 6 gets its last token
    pos = torch.arange(10, 10 + B, dtype=torch.int32)
    hlen = torch.arange(B, dtype=torch.int32)
    tok = torch.full((B,), 99, dtype=torch.long)
    out = torch.zeros(B, limit + 2, dtype=torch.long)
    n_hard, n_steps = torch.zeros((), dtype=torch.long), torch.zeros((), dtype=torch.long)
    d = lambda t: t.clone().to(dev)
    st = dict(hard_now=d(hard), phase=d(phase), tok=d(tok), finished=d(fin), pos=d(pos), out_tokens=d(out), out_len=d(out_len),
              hard_len=d(hlen), n_hard=d(n_hard), n_steps=d(n_steps))
    ops.greedy_tick(d(cur), d(prev), eos, limit, **st)
    both = (cur.float() + prev.float()).to(BF)
    want_tok = {2: int(cur[2].float().argmax()), 3: int(both[3].float().argmax()), 4: int(both[4].float().argmax()), 5: eos,
                6: int(cur[6].float().argmax())}
    got = {k: v.cpu() for k, v in st.items()}
    assert got["phase"].tolist() == [1, 0, 0, 0, 0, 0, 0]                     # row 0 moved on to its second iteration; row 1 untouched
    assert got["tok"].tolist() == [99, 99] + [want_tok[r] for r in range(2, 7)]
    assert got["pos"].tolist() == [10, 11, 13, 14, 15, 16, 17]
    assert got["out_len"].tolist() == [1, 2, 4, 2, 3, 2, limit]               # the end-of-sequence token is not written
    assert got["finished"].tolist() == [False, True, False, False, False, True, True]
    assert got["hard_len"].tolist() == [0, 1, 2, 4, 5, 5, 6]
    assert int(got["n_steps"]) == 5 and int(got["n_hard"]) == 2
    want_out = out.clone()
    for r, col in ((2, 3), (3, 1), (4, 2), (6, limit - 1)):
        want_out[r, col] = want_tok[r]
    assert torch.equal(got["out_tokens"], want_out)
    # tokens handed in instead of the arg-max (a sampled token): the same bookkeeping around them
    st = dict(hard_now=d(hard), phase=d(phase), tok=d(tok), finished=d(fin), pos=d(pos), out_tokens=d(out), out_len=d(out_len),
              hard_len=d(hlen), n_hard=d(n_hard), n_steps=d(n_steps))
    chosen = torch.tensor([70, 71, 72, 73, eos, 75, 76])
    ops.greedy_tick(d(cur), d(prev), eos, limit, chosen=d(chosen), **st)
    got = {k: v.cpu() for k, v in st.items()}
    assert got["tok"].tolist() == [99, 99, 72, 73, eos, 75, 76] and got["phase"].tolist() == [1, 0, 0, 0, 0, 0, 0]
    assert got["finished"].tolist() == [False, True, False, False, True, False, True]
    assert got["out_len"].tolist() == [1, 2, 4, 2, 2, 3, limit] and got["hard_len"].tolist() == [0, 1, 2, 4, 5, 5, 6]
    assert got["out_tokens"][2, 3] == 72 and got["out_tokens"][3, 1] == 73 and got["out_tokens"][5, 2] == 75 and got["out_tokens"][6, limit - 1] == 76


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_step_glue_on_cpu_shim():
    with emu_util.emulated():
        _step_begin_case("cpu")
        _step_begin_case("cpu", B=33, H=72, packed=False)   # more than 32 rows: no packed form
        _decider_tail_case("cpu")
        _step_begin_phase_case("cpu")
        _greedy_tick_case("cpu")


@pytest.mark.gpu
def test_step_glue_gpu():
    _step_begin_case("cuda", B=32, H=2048, V=5000, L=1600)
    _step_begin_case("cuda", B=40, H=1000, V=777, L=64, packed=False)
    _decider_tail_case("cuda", B=32, W=512)
    _decider_tail_case("cuda", B=7, W=2048)
    _step_begin_phase_case("cuda")
    _greedy_tick_case("cuda")
    _greedy_tick_case("cuda", V=151936)
