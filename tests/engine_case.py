"""The decode engine (tah_amd.engine) against the reference's forward loop restated around a Hugging Face
``Qwen3Model``: dense additive masks (oracle.duo_oracle.build_attention_mask = tah_model.py:744-791), a cache
that returns the concatenated K/V (oracle.duo_oracle.OracleCache = causal_cache.py:63-109), ``gather_active`` /
``scatter_back`` packing, the top-k softmax mix and the running sum of logits (tah_model.py:57-83, 580-706), in
float32 on the host.  Both sides are fed the same tokens and the same hard decisions (teacher forcing), so the
comparison is of logits, step by step, not of trajectories."""
import pytest
import torch

from oracle import duo_oracle as O


class _Cache(O.OracleCache):
    """What transformers' model code asks of a cache object besides update()."""

    def get_seq_length(self, layer_idx=0):
        return sum(t.shape[-2] for t in self.k.get((layer_idx, 0), []))

    def get_mask_sizes(self, cache_position, layer_idx):
        return cache_position.shape[0] + self.get_seq_length(layer_idx), 0


def _ref_forward(model, embed, cache, ids, valid, hard, topk, decide=None, mix_from_bf16_logits=False):
    """tah_model.py:495-706 for max_iter = 2 with the decider's decisions given: returns final logits (B, T, V).
    ``decide(logits, stacked hidden states (B, T, L + 1, H))``, when given, is called as the loop calls its decider after
    the first iteration (tah_model.py:434-441, 636-642) and its result returned as well."""
    B, T = ids.shape
    x = embed[ids]
    cached_valid = cache.get_valid_mask_upto_iter(0, 0, B)
    pos = (torch.cumsum(torch.cat((cached_valid, valid), -1), -1)[:, -T:] - 1).clamp(min=0)  # tah_model.py:555-561
    m0 = O.build_attention_mask(pos, valid, cache, 0, torch.float32)
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
    out0 = model(inputs_embeds=x, attention_mask={"full_attention": m0}, position_ids=pos, past_key_values=cache,
                 use_cache=True, output_hidden_states=decide is not None)
    h = out0.last_hidden_state
    cum = h @ embed.t()
    decided = decide(cum, torch.stack(list(out0.hidden_states), dim=0).permute(1, 2, 0, 3)) if decide is not None else None
    final = cum.clone()
    cur = hard & (valid == 1)
    if cur.any():
        pad, a_cum, a_pos, a_valid = O.gather_active(cur, cum, pos, valid)
        k = min(topk, a_cum.shape[-1])
        # (mix_from_bf16_logits: the first iteration's logits as a bf16 model holds them, for the top-k mix only)
        tv, ti = torch.topk(a_cum.to(torch.bfloat16).float() if mix_from_bf16_logits else a_cum, k=k, dim=-1)
        a_x = torch.sum(torch.softmax(tv, -1).unsqueeze(-1) * embed[ti], dim=-2)  # tah_model.py:57-75
        m1 = O.build_attention_mask(a_pos, a_valid, cache, 1, torch.float32)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 1, a_pos, a_valid
        h1 = model(inputs_embeds=a_x, attention_mask={"full_attention": m1}, position_ids=a_pos, past_key_values=cache,
                   use_cache=True).last_hidden_state
        final = O.scatter_back(cur, a_cum + h1 @ embed.t(), final)  # additive_logits_update, tah_model.py:78-83
    return final if decide is None else (final, decided)


def run(device, *, prompt=(9, 6, 12), steps=5, layers=2, seed=0, vocab=96, topk=100, hidden=256, hq=4, hkv=2,
        intermediate=512, decider_hidden=32, ref_device="cpu", with_hard=False, p_hard=0.35):
    """``ref_device``: where the float32 reference model and its dense logits live (the host by default; the
    end-to-end workload's own shape -- 28 layers, hidden 2048, 151 936 tokens -- wants the device).  ``with_hard``: every
    stage comes back as (engine logits, reference logits, which rows took the second iteration)."""
    pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    from transformers import Qwen3Config, Qwen3Model

    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights

    torch.manual_seed(seed)
    hf = Qwen3Config(hidden_size=hidden, num_attention_heads=hq, num_key_value_heads=hkv, head_dim=128,
                     num_hidden_layers=layers, intermediate_size=intermediate, vocab_size=vocab, rope_theta=1e6,
                     attention_dropout=0.0, rms_norm_eps=1e-6)
    hf._attn_implementation = "sdpa"
    with torch.device(ref_device):
        ref = Qwen3Model(hf)
    inv_freq = ref.rotary_emb.inv_freq.clone()
    ref = ref.to(torch.bfloat16).float().eval()  # bf16-representable weights, float32 arithmetic
    # (the round trip also rounds the rotary frequencies, a float32 buffer of the module, to bf16: angles would then be
    # off in proportion to the position -- 0.5 rad at position 480 -- which a short prompt hides and a long one does not)
    ref.rotary_emb.inv_freq.copy_(inv_freq)
    if hasattr(ref.rotary_emb, "original_inv_freq"):
        ref.rotary_emb.original_inv_freq = inv_freq.clone()
    cfg = EngineConfig(hidden=hidden, layers=layers, hq=hq, hkv=hkv, head_dim=128, intermediate=intermediate, vocab=vocab,
                       decider_hidden=decider_hidden, topk=topk)

    class _LM:  # the pieces Weights.from_hf reads: tied output head
        model = ref
        lm_head = type("H", (), {"weight": ref.embed_tokens.weight})
    w = Weights.from_hf(_LM, cfg, device)
    g = torch.Generator().manual_seed(seed + 1)
    w.dec_w1 = torch.randn(decider_hidden, hidden, generator=g).to(torch.bfloat16).to(device)
    w.dec_b1 = torch.zeros(decider_hidden, dtype=torch.bfloat16, device=device)
    w.dec_w2 = torch.randn(1, decider_hidden, generator=g).to(torch.bfloat16).to(device)
    w.dec_b2 = torch.zeros(1, dtype=torch.bfloat16, device=device)

    B, Tm = len(prompt), max(prompt)
    eng = TaHDecodeEngine(w, B, Tm + steps + 4, device=device)
    ids = torch.randint(0, vocab, (B, Tm + steps), generator=g)
    valid = torch.zeros(B, Tm, dtype=torch.long)
    for b, n in enumerate(prompt):
        valid[b, Tm - n:] = 1  # left padding, as the reference batches prompts
    hard = torch.rand(B, Tm + steps, generator=g) < p_hard
    hard[:, Tm] = torch.tensor([True] + [False] * (B - 1))   # first decode step: one hard row, the rest pad rows
    hard[:, Tm + 1] = False                                  # second: nobody iterates
    hard[:, Tm + 2] = True                                   # third: every row does
    hard[0, Tm - 1] = True                                   # a prompt whose last token is hard
    embed = ref.embed_tokens.weight.detach()
    rd = lambda t: t.to(ref_device)

    out = []
    with torch.no_grad():
        cache = _Cache()
        with torch.device(ref_device):  # (the oracle's helpers create their tensors on the default device)
            want = _ref_forward(ref, embed, cache, rd(ids[:, :Tm]), rd(valid), rd(hard[:, :Tm]), topk)[:, -1].cpu()
        packed = torch.cat([ids[b, Tm - n:Tm] for b, n in enumerate(prompt)]).to(device)
        hard_packed = torch.cat([hard[b, Tm - n:Tm] for b, n in enumerate(prompt)]).to(device)
        cu = torch.tensor([0] + list(torch.tensor(prompt).cumsum(0)), dtype=torch.int32, device=device)
        got, _ = eng.prefill(packed, cu, force_hard=hard_packed)
        out.append((got.cpu(), want) + ((hard[:, Tm - 1].clone(),) if with_hard else ()))
        one = rd(torch.ones(B, 1, dtype=torch.long))
        for s in range(steps):
            t = Tm + s
            with torch.device(ref_device):
                want = _ref_forward(ref, embed, cache, rd(ids[:, t:t + 1]), one, rd(hard[:, t:t + 1]), topk)[:, 0].cpu()
            got, h = eng.step_logits(ids[:, t].to(device), force_hard=hard[:, t].to(device))
            eng.pos += 1
            assert torch.equal(h.cpu(), hard[:, t])
            out.append((got.cpu(), want) + ((hard[:, t].clone(),) if with_hard else ()))
    lens0 = [n + steps for n in prompt]
    assert all(sl.len.tolist() == lens0 for sl in eng.slabs0)
    n1 = [int(hard[b, Tm - n:].sum()) for b, n in enumerate(prompt)]
    assert all(sl.len.tolist() == n1 for sl in eng.slabs1)
    return out


def run_greedy(device, *, fused, eos, B=3, T=9, new=7, vocab=64, seed=5, layers=2):
    """Greedy generation with the fused arg-max + bookkeeping step on or off; returns everything the loop leaves
    behind (tokens, lengths, positions, finished flags, counters, slab lengths)."""
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights

    cfg = EngineConfig(hidden=256, layers=layers, hq=4, hkv=2, head_dim=128, intermediate=512, vocab=vocab, decider_hidden=32)
    w = Weights.random_init(cfg, device, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    ids = torch.randint(0, vocab, (B * T,), generator=g).to(device)
    cu = torch.arange(0, B * T + 1, T, dtype=torch.int32, device=device)
    eng = TaHDecodeEngine(w, B, T + new + 2, device=device)
    eng.fused_greedy = fused
    first, _ = eng.prefill(ids, cu, calibrate=0.3)
    toks = eng.generate(first, new, eos=eos, use_graph=False).clone()
    return (toks.cpu(), eng.out_len.cpu(), eng.pos.cpu(), eng.finished.cpu(), int(eng.n_hard), int(eng.n_steps), eng.tok.cpu(),
            [sl.len.tolist() for sl in eng.slabs0 + eng.slabs1])


def run_with_decider(device, *, prompt=(9, 6, 12), steps=4, layers=3, seed=2, vocab=96):
    """The engine deciding with tah_amd.decider.MLPIterDecider: the decision logits it computes in prefill (every
    prompt token) and in every decode step against oracle/decider_ref.py fed with the Hugging Face model's own
    logits and ``output_hidden_states`` (float32), both sides driven by the same tokens and decisions.  Returns
    pairs (engine's decision logits, oracle's) per call."""
    pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    from transformers import Qwen3Config, Qwen3Model

    from oracle import decider_ref as R
    from tah_amd.decider import MLPIterDecider
    from tah_amd.engine import EngineConfig, TaHDecodeEngine, Weights
    from tests import decider_case as D

    torch.manual_seed(seed)
    hf = Qwen3Config(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
                     num_hidden_layers=layers, intermediate_size=512, vocab_size=vocab, rope_theta=1e6,
                     attention_dropout=0.0, rms_norm_eps=1e-6)
    hf._attn_implementation = "sdpa"
    ref = Qwen3Model(hf)
    inv_freq = ref.rotary_emb.inv_freq.clone()
    ref = ref.to(torch.bfloat16).float().eval()
    ref.rotary_emb.inv_freq.copy_(inv_freq)  # (a float32 buffer the round trip must not round, see run())
    cfg = EngineConfig(hidden=256, layers=layers, hq=4, hkv=2, head_dim=128, intermediate=512, vocab=vocab,
                       decider_hidden=32, topk=100)

    class _LM:
        model = ref
        lm_head = type("H", (), {"weight": ref.embed_tokens.weight})
    w = Weights.from_hf(_LM, cfg, device)
    picks = (1, layers)   # after the first layer, and the last one (after the final norm)
    dec = D.make(device, torch.bfloat16, seed=seed + 3, topk=10, hidden_states_size=256, hidden_states_layer_nums=picks,
                 hidden_dims=(32, 64, 32), expansion_factor=2)  # (widths the linear-layer kernel takes)
    p64 = D.state64(dec)

    def decide(logits, stack):
        return torch.from_numpy(R.decide(p64, logits.numpy(), 1, stack.numpy(), topk=10, hidden_size=256, layer_nums=picks,
                                         n_blocks=3, max_iter=3)[1])

    g = torch.Generator().manual_seed(seed + 1)
    B, Tm = len(prompt), max(prompt)
    eng = TaHDecodeEngine(w, B, Tm + steps + 4, device=device, decider=dec)
    ids = torch.randint(0, vocab, (B, Tm + steps), generator=g)
    valid = torch.zeros(B, Tm, dtype=torch.long)
    for b, n in enumerate(prompt):
        valid[b, Tm - n:] = 1
    hard = torch.rand(B, Tm + steps, generator=g) < 0.35
    embed = ref.embed_tokens.weight.detach()
    out = []
    with torch.no_grad():
        cache = _Cache()
        _, z = _ref_forward(ref, embed, cache, ids[:, :Tm], valid, hard[:, :Tm], 100, decide)
        packed = torch.cat([ids[b, Tm - n:Tm] for b, n in enumerate(prompt)]).to(device)
        hard_packed = torch.cat([hard[b, Tm - n:Tm] for b, n in enumerate(prompt)]).to(device)
        cu = torch.tensor([0] + list(torch.tensor(prompt).cumsum(0)), dtype=torch.int32, device=device)
        eng.prefill(packed, cu, force_hard=hard_packed)
        out.append((eng.decision_logits.float().cpu(), torch.cat([z[b, Tm - n:] for b, n in enumerate(prompt)])))
        one = torch.ones(B, 1, dtype=torch.long)
        for s_ in range(steps):
            t = Tm + s_
            _, z = _ref_forward(ref, embed, cache, ids[:, t:t + 1], one, hard[:, t:t + 1], 100, decide)
            eng.step_logits(ids[:, t].to(device), force_hard=hard[:, t].to(device))
            eng.pos += 1
            out.append((eng.decision_logits.float().cpu(), z[:, 0]))
    return out

