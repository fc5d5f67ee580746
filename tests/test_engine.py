"""Decode engine: the iteration loop for one token per sequence on the native kernels."""
import pytest
import torch

from tests import emu_util


def _check(outs):
    for i, (got, want) in enumerate(outs):
        err = (got - want).abs().max().item()
        ref = want.abs().max().item()
        assert err <= 3e-2 * max(ref, 1.0), (i, err, ref)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_engine_matches_reference_loop_on_cpu_shim():
    from tests.engine_case import run
    with emu_util.emulated():
        _check(run("cpu", prompt=(7, 4), steps=3))  # one hard row and a pad row, nobody, everybody


def _same_greedy(device, **size):
    from tests.engine_case import run_greedy
    same = lambda a, b, e: [None for x, y in zip(a, b) if not (torch.equal(x, y) if torch.is_tensor(x) else x == y)] == [] or \
        pytest.fail(f"fused and plain greedy steps differ (eos={e}): {a} vs {b}")
    plain = run_greedy(device, fused=False, eos=-1, **size)
    same(plain, run_greedy(device, fused=True, eos=-1, **size), -1)
    # an end-of-sequence token that the run is known to produce part-way for some row: rows finish at different steps
    eos = int(plain[0][0, 2])
    a = run_greedy(device, fused=False, eos=eos, **size)
    same(a, run_greedy(device, fused=True, eos=eos, **size), eos)
    assert bool(a[3].any())  # some row did finish


def _greedy_step_case(device, rows=6, vocab=200, seed=0):
    """ops.greedy_step against the engine's own torch bookkeeping (engine.py:_step_inplace) on random logits with
    ties, rows already finished, rows that hit the end-of-sequence token and rows that took a second iteration."""
    from tah_amd import ops
    g = torch.Generator().manual_seed(seed)
    padded = (vocab + 7) // 8 * 8  # rows start on 16-byte boundaries; the vocabulary itself may be any size
    l0p = (torch.randn(rows, padded, generator=g) * 3).to(torch.bfloat16)
    l1p = (torch.randn(rows, padded, generator=g) * 3).to(torch.bfloat16)
    l0, l1 = l0p[:, :vocab], l1p[:, :vocab]
    l0[1, 7] = l0[1, 150] = 40.0               # a tie at the maximum: the lower index wins
    hard = torch.tensor([False, False, True, True, False, True])[:rows]
    finished = torch.tensor([False, False, False, True, False, False])[:rows]
    final = torch.where(hard[:, None], (l0 + l1).float(), l0.float())
    eos = int(final[4].argmax())               # row 4 produces the end-of-sequence token at this step
    st = dict(tok=torch.full((rows,), 5, dtype=torch.long), finished=finished.clone(), pos=torch.arange(10, 10 + rows, dtype=torch.int32),
              out_tokens=torch.zeros(rows, 4, dtype=torch.long), step_idx=torch.tensor([2]), out_len=torch.full((rows,), 2, dtype=torch.int32),
              n_hard=torch.tensor(3), n_steps=torch.tensor(11))
    dev = {k: v.clone().to(device) for k, v in st.items()}
    ops.greedy_step(l0p.to(device)[:, :vocab], l1p.to(device)[:, :vocab], (hard & ~finished).to(device), eos, dev["tok"], dev["finished"], dev["pos"],
                    dev["out_tokens"], dev["step_idx"], dev["out_len"], dev["n_hard"], dev["n_steps"])
    # the same step as the unfused loop writes it
    act = ~st["finished"]
    nxt = torch.where(act, final.argmax(-1), torch.zeros(rows, dtype=torch.long))
    assert int(nxt[1]) == 7
    st["finished"] |= nxt == eos
    keep = ~st["finished"]
    st["out_tokens"][:, 2] = torch.where(keep, nxt, torch.zeros_like(nxt))
    st["out_len"] += keep.to(torch.int32)
    st["n_hard"] += (hard & act).sum()
    st["n_steps"] += act.sum()
    st["pos"] += act.to(torch.int32)
    st["tok"] = nxt
    for k in st:
        assert torch.equal(dev[k].cpu(), st[k]), k
    # a step beyond the last column of out_tokens (a captured step replayed too often) stores nothing and ends the rows
    dev["step_idx"].fill_(4)
    before = dev["out_tokens"].clone()
    ops.greedy_step(l0p.to(device)[:, :vocab], None, None, -1, dev["tok"], dev["finished"], dev["pos"],
                    dev["out_tokens"], dev["step_idx"], dev["out_len"], dev["n_hard"], dev["n_steps"])
    assert torch.equal(dev["out_tokens"], before) and bool(dev["finished"].all())
    assert torch.equal(dev["out_len"].cpu(), st["out_len"])


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_greedy_step_kernel_on_cpu_shim():
    with emu_util.emulated():
        _greedy_step_case("cpu")
        _greedy_step_case("cpu", vocab=203, seed=1)   # a vocabulary that is not a multiple of 8


@pytest.mark.gpu
def test_greedy_step_kernel_gpu():
    _greedy_step_case("cuda", vocab=151936)
    _greedy_step_case("cuda", vocab=1003, seed=2)


@pytest.mark.gpu
def test_fused_greedy_step_equals_the_torch_bookkeeping_gpu():
    _same_greedy("cuda")


@pytest.mark.gpu
def test_engine_matches_reference_loop_gpu():
    from tests.engine_case import run
    _check(run("cuda", prompt=(40, 23, 64), steps=6))


@pytest.mark.gpu
def test_engine_topk_smaller_than_vocab_gpu():
    from tests.engine_case import run
    # a sharper top-k (k < vocab): ties at the k-th logit may be broken differently by the two sides, so the
    # bound is looser; what it guards is the k < V code path end to end
    for got, want in run("cuda", prompt=(30, 31), steps=4, vocab=512, topk=100, seed=3):
        err = (got - want).abs().max().item()
        assert err <= 6e-2 * max(want.abs().max().item(), 1.0)


@pytest.mark.gpu
def test_engine_graph_replay_equals_eager_gpu():
    """The captured step replayed N times gives the tokens, lengths and counters of N eager steps (every replay
    is checked, with eager work and synchronisation in between)."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    cfg = EngineConfig(hidden=256, layers=2, hq=4, hkv=2, head_dim=128, intermediate=512, vocab=5000, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=4)
    B, T, new = 4, 33, 12
    g = torch.Generator().manual_seed(9)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    runs = []
    for use_graph in (False, True):
        eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
        first, hard = eng.prefill(ids, cu, calibrate=0.3)
        if not use_graph:
            toks = eng.generate(first, new, use_graph=False).clone()
            per_step = None
        else:
            # step by step: replay, synchronise, run some eager work, compare the column just written
            eng.out_tokens.zero_(); eng.step_idx.zero_()
            f = eng.sample(first, 0.0)
            eng.out_tokens[:, 0] = f; eng.tok.copy_(f); eng.step_idx += 1
            gr = eng.capture(0.0, -1)
            for s in range(1, new):
                gr.replay()
                torch.cuda.synchronize()
                _ = (torch.randn(64, 64, device="cuda") @ torch.randn(64, 64, device="cuda")).sum().item()
                assert torch.equal(eng.out_tokens[:, s], runs[0][0][:, s]), f"replay {s} differs from the eager step"
            toks = eng.out_tokens[:, :new].clone()
        runs.append((toks, int(eng.n_hard), [sl.len.tolist() for sl in eng.slabs0 + eng.slabs1], eng.pos.tolist()))
    assert torch.equal(runs[0][0], runs[1][0]) and runs[0][1:] == runs[1][1:]
    assert runs[0][1] > 0  # some token took the second iteration


def test_sampling_filters_follow_the_reference_semantics():
    """``TaHDecodeEngine.sample`` against the rules of ``sample_next_token`` (tah/model/utils.py:84-125): arg-max
    when not sampling; min_p / top_k / top_p each confine the draw to the set the rule names."""
    from tah_amd.engine import TaHDecodeEngine as E
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(6, 50, generator=g) * 2
    am = logits.argmax(-1)
    assert torch.equal(E.sample(logits, 0.0), am)
    torch.manual_seed(1)
    for kw in (dict(top_k=1), dict(min_p=1.0), dict(top_p=1e-6)):
        assert torch.equal(E.sample(logits, 0.7, **kw), am), kw
    probs = torch.softmax(logits / 0.7, -1)
    top3 = probs.topk(3, -1).indices
    sp, si = probs.sort(descending=True, dim=-1)
    # top_p = 0.5: the smallest prefix of the sorted distribution whose mass reaches 0.5
    npfx = ((sp.cumsum(-1) - sp) < 0.5).sum(-1)
    seen_k, seen_p = set(), set()
    for _ in range(300):
        a = E.sample(logits, 0.7, top_k=3)
        assert all(a[r] in top3[r] for r in range(6))
        seen_k.add(int(a[0]))
        b = E.sample(logits, 0.7, top_p=0.5)
        assert all(b[r] in si[r, : int(npfx[r])] for r in range(6))
        c = E.sample(logits, 0.7, min_p=0.3)
        assert all(probs[r, c[r]] >= 0.3 * probs[r].max() for r in range(6))
    assert len(seen_k) > 1  # it does sample
    # the draw follows the distribution: frequencies of a 3-way choice within 4 sigma
    lg = torch.log(torch.tensor([[0.6, 0.3, 0.1]])).expand(4000, 3)
    freq = torch.bincount(E.sample(lg, 1.0), minlength=3).float() / 4000
    assert (freq - torch.tensor([0.6, 0.3, 0.1])).abs().max() < 4 * (0.25 / 4000) ** 0.5


@pytest.mark.gpu
def test_generate_wrapper_returns_tokens_up_to_eos_gpu():
    """``tah_amd.engine.generate`` (the call signature and return value of TaHForCasualLM_generate): greedy tokens
    equal the engine's own stepping; with an end-of-sequence id a row's list stops before it, other rows go on."""
    import types

    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights, generate
    cfg = EngineConfig(hidden=256, layers=2, hq=4, hkv=2, head_dim=128, intermediate=512, vocab=304, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=5)
    B, T, new = 3, 20, 24
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, cfg.vocab, (B, T), generator=g).cuda()
    mask = torch.ones(B, T, dtype=torch.long, device="cuda")
    mask[1, :6] = 0  # a left-padded prompt
    tok = types.SimpleNamespace(eos_token_id=None, decode=lambda t: " ".join(map(str, t)))
    w.threshold = 0.45
    free, texts = generate(TaHDecodeEngine(w, B, T + new + 2), tok, dict(input_ids=ids, attention_mask=mask),
                           max_new_tokens=new, do_sample=False)
    assert [len(t) for t in free] == [new] * B and texts[0] == " ".join(map(str, free[0]))
    eager, _ = generate(TaHDecodeEngine(w, B, T + new + 2), tok, dict(input_ids=ids, attention_mask=mask),
                        max_new_tokens=new, do_sample=False, use_graph=False)
    assert eager == free
    tok.eos_token_id = free[0][5]
    cut, _ = generate(TaHDecodeEngine(w, B, T + new + 2), tok, dict(input_ids=ids, attention_mask=mask),
                      max_new_tokens=new, do_sample=False)
    for b in range(B):
        stop = free[b].index(tok.eos_token_id) if tok.eos_token_id in free[b] else new
        assert cut[b] == free[b][:stop], b
    assert len(cut[0]) <= 5


@pytest.mark.gpu
def test_engine_with_fused_layer_attention_equals_the_separate_launches_gpu():
    """32 sequences x 8 kv heads: the engine runs q/k preparation, append and attention of a layer in one launch
    (tah_duo_decode_step).  Driven with the same tokens and hard decisions, it gives the logits of the separate
    launches (to the last bits of bf16: the two kernels are compiled separately) and exactly their cache lengths; its
    captured step gives exactly the tokens of its eager step."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    cfg = EngineConfig(hidden=256, layers=2, hq=16, hkv=8, head_dim=128, intermediate=768, vocab=4096, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=6)
    B, T, steps = 32, 21, 5
    g = torch.Generator().manual_seed(10)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    toks = torch.randint(0, cfg.vocab, (steps, B), generator=g).cuda()
    hards = (torch.rand(steps, B, generator=g) < 0.3).cuda()
    hards[1], hards[2] = False, True
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    runs = []
    for fused in (False, True):
        eng = TaHDecodeEngine(w, B, T + steps + 12, device="cuda")
        assert eng.fused_step and eng.packed_linear
        eng.fused_step = fused
        eng.prefill(ids, cu, calibrate=0.2)
        logits = []
        for s in range(steps):
            got, h = eng.step_logits(toks[s], force_hard=hards[s])
            eng.pos += 1
            logits.append(got)
        runs.append((logits, [sl.len.tolist() for sl in eng.slabs0 + eng.slabs1], eng.hard_len.tolist()))
    for a, b in zip(runs[0][0], runs[1][0]):
        assert (a - b).abs().max().item() <= 2e-2 * max(a.abs().max().item(), 1.0)
    assert runs[0][1:] == runs[1][1:]
    assert runs[1][2] == runs[1][1][cfg.layers]  # the engine's own count of depth-1 rows is what the slabs hold
    # the fused step under the graph: the tokens of its eager run
    out = []
    for use_graph in (False, True):
        eng = TaHDecodeEngine(w, B, T + 12, device="cuda")
        first, _ = eng.prefill(ids, cu, calibrate=0.2)
        out.append((eng.generate(first, 10, eos=7, use_graph=use_graph).clone(), int(eng.n_hard), eng.hard_len.tolist(),
                    [sl.len.tolist() for sl in eng.slabs0 + eng.slabs1]))
    assert torch.equal(out[0][0], out[1][0]) and out[0][1:] == out[1][1:] and out[0][1] > 0


@pytest.mark.gpu
def test_engine_fused_glue_agrees_with_the_torch_glue_gpu():
    """One step from the same state through tah_step_begin / the decider on the linear-layer kernel / tah_decider_tail
    and through the torch operations they replace: the first iteration's logits are the same launches on the same
    inputs (equal), the decisions agree except where a probability sits within rounding of the threshold, and the
    second iteration's logits agree for rows both call hard."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    cfg = EngineConfig(hidden=256, layers=2, hq=4, hkv=2, head_dim=128, intermediate=512, vocab=4096, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=8)
    B, T = 16, 19
    g = torch.Generator().manual_seed(12)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    outs = []
    for fused in (True, False):
        eng = TaHDecodeEngine(w, B, T + 8, device="cuda")
        assert eng.fused_glue
        eng.use_fused_glue = fused
        first, _ = eng.prefill(ids, cu, calibrate=0.3)
        eng.tok.copy_(first.argmax(-1))
        eng.finished[3] = True
        l0, l1, hard, _ = eng._parts()
        outs.append((l0.float().clone(), l1.float().clone(), hard.clone(), [sl.len.tolist() for sl in eng.slabs0]))
    (a0, a1, ha, la), (b0, b1, hb, lb) = outs
    assert torch.equal(a0, b0) and la == lb
    assert (ha == hb).float().mean() >= 0.9 and ha.any() and not ha[3]
    both = ha & hb
    assert (a1[both] - b1[both]).abs().max().item() <= 2e-2 * max(b1[both].abs().max().item(), 1.0)


@pytest.mark.gpu
def test_engine_beyond_32_rows_falls_back_to_library_gemms_gpu():
    """33 sequences: the linear-layer kernels take at most 32 rows, so the step runs on torch GEMMs and the torch glue;
    the captured step still gives the eager step's tokens, and the first 32 rows' prefill logits do not depend on the
    33rd sequence being there."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    cfg = EngineConfig(hidden=256, layers=2, hq=4, hkv=2, head_dim=128, intermediate=512, vocab=2048, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=9)
    B, T, new = 33, 17, 6
    g = torch.Generator().manual_seed(13)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    out = []
    for use_graph in (False, True):
        eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
        assert not eng.packed_linear and not eng.fused_glue and not eng.fused_step
        first, _ = eng.prefill(ids, cu, calibrate=0.3)
        out.append((first.clone(), eng.generate(first, new, use_graph=use_graph).clone(), int(eng.n_hard)))
    assert torch.equal(out[0][1], out[1][1]) and out[0][2] == out[1][2] and out[0][2] > 0
    small = TaHDecodeEngine(w, 32, T + new + 2, device="cuda")
    assert small.packed_linear
    first32, _ = small.prefill(ids[:32 * T], cu[:33])
    assert torch.allclose(first32, out[0][0][:32], atol=2e-2 * float(first32.abs().max()))


@pytest.mark.gpu
def test_engine_can_be_used_for_a_second_batch_gpu():
    """prefill() starts from empty slabs: a second generation on the same engine equals the first one and a fresh
    engine's."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    cfg = EngineConfig(hidden=256, layers=2, hq=4, hkv=2, head_dim=128, intermediate=512, vocab=2048, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=11)
    B, T, new = 4, 15, 8
    g = torch.Generator().manual_seed(14)
    ids = torch.randint(0, cfg.vocab, (2, B * T), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
    runs = []
    for which in (0, 1, 0):
        first, _ = eng.prefill(ids[which], cu, calibrate=None)
        runs.append((eng.generate(first, new).clone(), int(eng.n_hard), [sl.len.tolist() for sl in eng.slabs0 + eng.slabs1]))
    assert torch.equal(runs[0][0], runs[2][0]) and runs[0][1:] == runs[2][1:]
    assert not torch.equal(runs[0][0], runs[1][0])
    fresh = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
    first, _ = fresh.prefill(ids[1], cu)
    assert torch.equal(fresh.generate(first, new), runs[1][0])


@pytest.mark.gpu
@pytest.mark.parametrize("eos", [-1, 7])
def test_continuous_generation_gives_the_tokens_of_the_stepwise_loop_gpu(eos):
    """Rows at different latent iterations in one batch (generate(continuous=True)) against the loop that keeps the
    batch in step: rows do not interact, so tokens, lengths, counters and cache lengths have to be the same; the ticks
    needed are fewer than two per token."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    cfg = EngineConfig(hidden=256, layers=2, hq=16, hkv=8, head_dim=128, intermediate=768, vocab=4096, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=6)
    B, T, new = 32, 21, 24
    g = torch.Generator().manual_seed(10)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    runs = []
    for continuous, use_graph in ((False, True), (True, False), (True, True)):
        eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
        assert eng.can_run_continuous
        first, _ = eng.prefill(ids, cu, calibrate=0.25)
        toks = eng.generate(first, new, eos=eos, continuous=continuous, use_graph=use_graph).clone()
        n_out = eng.out_len.clone()
        live = torch.arange(new, device="cuda")[None, :] < n_out[:, None]
        runs.append((torch.where(live, toks, torch.zeros_like(toks)).cpu(), n_out.cpu(), eng.finished.cpu(), int(eng.n_hard),
                     [sl.len.tolist() for sl in eng.slabs1], getattr(eng, "ticks", None)))
    ref = runs[0]
    assert 0 < ref[3]
    for r in runs[1:]:
        assert torch.equal(r[0], ref[0]) and torch.equal(r[1], ref[1]) and torch.equal(r[2], ref[2])
        assert r[3] == ref[3] and r[4] == ref[4]
        assert new - 1 <= r[5] <= 2 * (new - 1) + 8  # (the host looks every 8 ticks)


@pytest.mark.gpu
def test_continuous_generation_with_sampling_gpu():
    """Sampled tokens in ticks.  With a stand-in for the draw that is a function of the final logits alone (their
    second-largest entry) the tokens have to be those of the step-wise loop, eager and captured; with the real draw the
    generation runs to its length and every row gets its tokens."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    cfg = EngineConfig(hidden=256, layers=2, hq=16, hkv=8, head_dim=128, intermediate=768, vocab=4096, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=7)
    B, T, new = 32, 17, 20
    g = torch.Generator().manual_seed(11)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")

    def second_best(logits, temperature=0.0, **_):
        return torch.topk(logits, 2, dim=-1).indices[:, 1] if temperature > 0.0 else torch.argmax(logits, dim=-1)

    runs = []
    for continuous, use_graph in ((False, True), (True, False), (True, True)):
        eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
        eng.sample = second_best
        eng.fused_sampling = False  # (draws without a top-k filter go through ``sample``)
        first, _ = eng.prefill(ids, cu, calibrate=0.25)
        toks = eng.generate(first, new, temperature=0.7, eos=-1, continuous=continuous, use_graph=use_graph).clone()
        runs.append((toks.cpu(), eng.out_len.cpu(), int(eng.n_hard), [sl.len.tolist() for sl in eng.slabs1]))
    assert 0 < runs[0][2] and (runs[0][1] == new).all()
    for r in runs[1:]:
        assert torch.equal(r[0], runs[0][0]) and torch.equal(r[1], runs[0][1]) and r[2] == runs[0][2] and r[3] == runs[0][3]
    greedy = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
    first, _ = greedy.prefill(ids, cu, calibrate=0.25)
    assert not torch.equal(greedy.generate(first, new).cpu(), runs[0][0])   # (the stand-in was really used)
    eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
    first, _ = eng.prefill(ids, cu, calibrate=0.25)
    toks = eng.generate(first, new, temperature=0.8, top_p=0.9, top_k=50, eos=-1)   # ticks by default, captured
    assert eng.ticks >= new - 1 and (eng.out_len == new).all() and int(eng.n_steps) == B * (new - 1)
    assert int(toks.min()) >= 0 and int(toks.max()) < cfg.vocab
    top50 = torch.topk(first, 50, dim=-1).indices
    assert (toks[:, :1] == top50).any(dim=-1).all()                          # the first draw obeys the top-k filter
    # the same prompt in every row: the captured tick must draw anew at every replay and for every row
    same = ids[:T].repeat(B)
    eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
    first, _ = eng.prefill(same, cu, calibrate=0.25)
    toks = eng.generate(first, new, temperature=1.0, top_k=50, eos=-1)
    assert len({tuple(r.tolist()) for r in toks}) > B // 2
    assert min(len(set(toks[:, j].tolist())) for j in range(1, new)) > B // 4
    # without a top-k filter the draw is one tah_sample_rows launch on the tick's and the previous tick's logits.  With
    # top_p so small that only the largest token survives, it has to reproduce the greedy generation, step-wise and in ticks
    want = greedy.out_tokens[:, :new].cpu()
    for continuous in (False, True):
        eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
        first, _ = eng.prefill(ids, cu, calibrate=0.25)
        toks = eng.generate(first, new, temperature=0.9, top_p=1e-6, eos=-1, continuous=continuous)
        assert torch.equal(toks.cpu(), want), continuous
    # and with real filters: every row gets its tokens, equal rows draw apart, at every replay
    eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
    first, _ = eng.prefill(same, cu, calibrate=0.25)
    toks = eng.generate(first, new, temperature=1.0, top_p=0.95, min_p=0.001, eos=-1)
    assert eng.ticks >= new - 1 and (eng.out_len == new).all()
    assert int(toks.min()) >= 0 and int(toks.max()) < cfg.vocab
    assert len({tuple(r.tolist()) for r in toks}) > B // 2
    assert min(len(set(toks[:, j].tolist())) for j in range(1, new)) > B // 4


def _topk_sampling_case(device, V, rows=6, draws=True):
    """The distribution over the k largest logits that sample_topk draws from against the one the reference's filters
    leave on the whole row (utils.py:84-125), on rows without equal values; and the draws land where it is not zero."""
    from tah_amd import ops
    from tah_amd.engine import TaHDecodeEngine as E
    g = torch.Generator().manual_seed(V)
    # 300 different values from the bf16 grid of [1, 8) at random places (every filter's boundary falls among them),
    # the rest of the row below them
    grid = torch.arange(0x3F80, 0x4100, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    logits = (torch.rand(rows, V, generator=g) * 4 - 3.2).to(torch.bfloat16)
    for r in range(rows):
        logits[r, torch.randperm(V, generator=g)[:300]] = grid[torch.randperm(grid.numel(), generator=g)[:300]]
    logits = logits.to(device)
    for T, top_p, top_k, min_p in ((0.6, 0.95, 20, 0.0), (1.0, 1.0, 50, 0.0), (0.8, 0.7, 256, 0.05), (1.3, 0.9, 1, 0.0))[:4 if draws else 3]:
        want = E.filtered_probs(logits.float(), T, top_p=top_p, top_k=top_k, min_p=min_p)
        vals, idx = ops.topk(logits, top_k)
        got = torch.zeros_like(want).scatter_(1, idx.long(), E.topk_filtered_probs(vals, T, top_p=top_p, min_p=min_p))
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-7), float((got - want).abs().max())
        assert torch.equal(got > 0, want > 0)
        for _ in range(3 if draws else 1):
            tok = E.sample_topk(logits, T, top_p=top_p, top_k=top_k, min_p=min_p)
            assert tok.dtype == torch.int64 and (torch.gather(want, 1, tok[:, None]) > 0).all()
    if not draws:
        return
    # a draw follows the distribution: two tokens at 3:1
    two = torch.full((1, V), -30.0, dtype=torch.bfloat16, device=device)
    two[0, 5], two[0, 9] = 1.0986, 0.0
    draws = torch.stack([E.sample_topk(two.expand(64, V).contiguous(), 1.0, top_k=4) for _ in range(40)]).flatten()
    assert set(draws.tolist()) == {5, 9} and 0.70 < float((draws == 5).float().mean()) < 0.80


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_sampling_on_the_topk_values_on_cpu_shim():
    with emu_util.emulated():
        _topk_sampling_case("cpu", 3000, rows=2, draws=False)


@pytest.mark.gpu
def test_sampling_on_the_topk_values_gpu():
    _topk_sampling_case("cuda", 20000)


def _decider_wiring_check(device, **size):
    from tests import engine_case
    for got, want in engine_case.run_with_decider(device, **size):
        want = want.float()
        assert got.shape == want.shape
        err = (got - want).abs()
        # (bf16 model and decider against float32 / float64: measured 0.03 at most, 0.02 on average, on logits of size 2;
        # a wrong layer or a missing final norm moves them by their own size)
        assert float((err / (0.08 + 0.03 * want.abs())).max()) <= 1.0, (float(err.max()), float(want.abs().max()))
        assert float(err.mean()) <= 0.02 * float(want.abs().mean()) + 0.02


@pytest.mark.gpu
def test_engine_with_the_learned_decider_gpu():
    """The hidden states and logits the engine hands tah_amd.decider.MLPIterDecider are the ones the Hugging Face
    model reports with output_hidden_states (embeddings, after each layer, the last after the final norm).  (On the
    CPU execution build the same check takes a minute and a half; it is run by hand there:
    ``_decider_wiring_check("cpu", prompt=(3, 2), steps=1, layers=2)`` inside ``emu_util.emulated()``.)"""
    _decider_wiring_check("cuda")
    # and deciding by itself: ticks (eager and captured) give the step-wise loop's tokens
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    from tests import decider_case as D
    cfg = EngineConfig(hidden=256, layers=3, hq=16, hkv=8, head_dim=128, intermediate=768, vocab=4096, decider_hidden=32)
    w = Weights.random_init(cfg, "cuda", seed=8)
    dec = D.make("cuda", torch.bfloat16, seed=12, topk=10, hidden_states_size=256, hidden_states_layer_nums=(1, 2, 3),
                 hidden_dims=(32, 64, 32), expansion_factor=2)  # (widths the linear-layer kernel takes)
    B, T, new = 32, 19, 18
    g = torch.Generator().manual_seed(13)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    runs = []
    for continuous, use_graph in ((False, False), (False, True), (True, False), (True, True)):
        eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda", decider=dec)
        assert eng.can_run_continuous
        first, hard = eng.prefill(ids, cu, calibrate=0.25)
        toks = eng.generate(first, new, continuous=continuous, use_graph=use_graph).clone()
        runs.append((toks.cpu(), int(eng.n_hard), [sl.len.tolist() for sl in eng.slabs1], int(hard.sum())))
    assert 0 < runs[0][1] < B * (new - 1) and 0 < runs[0][3] < B * T
    for r in runs[1:]:
        assert torch.equal(r[0], runs[0][0]) and r[1:] == runs[0][1:]



@pytest.mark.gpu
def test_engine_at_the_end_to_end_shape_gpu():
    """The end-to-end workload's own shape (``EngineConfig()``: 28 layers, hidden 2048, 16 / 8 heads, 151 936 tokens;
    32 prompts of 512 tokens), where the other engine tests use a model a hundred times smaller:
    (a) greedy generation in captured ticks, in eager ticks and in the captured step-wise loop gives the same tokens,
    lengths, hard counts and slab lengths;
    (b) the prefill's and three decode steps' final logits (a step with a single hard row and pad rows, one with none, one
    where every row iterates) against the reference's loop around a float32 transformers ``Qwen3Model`` with dense masks
    and a concatenating cache, same tokens and hard decisions on both sides.  Rows that take one iteration: within 3e-2 of
    the logits' range, the bound of the small-model tests (bf16 weights, activations and logits through 28 layers on one
    side, float32 on the other).  Rows that take the second iteration get a loose bound (mean 6e-2, largest 0.4 of the
    range): their input is a softmax over the top-100 first-iteration logits, which turns a logit difference of one bf16
    step into a few per cent of weight, and 28 randomly initialised layers carry that on -- the float32 reference alone
    moves by 0.3 (hidden 2048, two layers, range 12.8) when only its own logits are rounded to bf16 before the mix."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    from tests.engine_case import run
    cfg = EngineConfig()
    w = Weights.random_init(cfg, "cuda", seed=11)
    B, T, new = 32, 512, 6
    g = torch.Generator().manual_seed(12)
    ids = torch.randint(0, cfg.vocab, (B * T,), generator=g).cuda()
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device="cuda")
    runs = []
    for continuous, use_graph in ((False, True), (True, False), (True, True)):
        eng = TaHDecodeEngine(w, B, T + new + 2, device="cuda")
        assert eng.can_run_continuous
        first, _ = eng.prefill(ids, cu, calibrate=0.25)
        toks = eng.generate(first, new, continuous=continuous, use_graph=use_graph).clone()
        runs.append((toks.cpu(), eng.out_len.cpu(), int(eng.n_hard), [sl.len.tolist() for sl in eng.slabs0 + eng.slabs1]))
        del eng
    assert 0 < runs[0][2] and (runs[0][1] == new).all()
    for r in runs[1:]:
        assert torch.equal(r[0], runs[0][0]) and torch.equal(r[1], runs[0][1]) and r[2] == runs[0][2] and r[3] == runs[0][3]
    del w, runs
    torch.cuda.empty_cache()
    prompts = tuple([512] * 29 + [500, 384, 77])
    plain, second = 0.0, (0.0, 0.0)
    for got, want, hard in run("cuda", prompt=prompts, steps=3, layers=cfg.layers, seed=13, vocab=cfg.vocab, topk=cfg.topk, hidden=cfg.hidden,
                               hq=cfg.hq, hkv=cfg.hkv, intermediate=cfg.intermediate, decider_hidden=cfg.decider_hidden, ref_device="cuda",
                               with_hard=True):
        rng = max(want.max().item() - want.min().item(), 1e-6)
        d = (got.float() - want).abs()
        if (~hard).any():
            plain = max(plain, d[~hard].max().item() / rng)
        if hard.any():
            second = (max(second[0], d[hard].max().item() / rng), max(second[1], d[hard].mean().item() / rng))
    print(f"end-to-end shape, error / logit range: rows with one iteration max {plain:.3e}; rows with two: max {second[0]:.3e}, "
          f"mean {second[1]:.3e}", flush=True)
    assert plain <= 3e-2 and second[0] <= 0.4 and second[1] <= 6e-2
