"""A transformers Qwen3Attention module run twice on the same input: its own forward (eager bf16 modules,
SDPA with the dense additive mask the reference would build) and this library's fused forward."""
import pytest
import torch


def run(device, B=2, T=37, seed=0):
    m = pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    from transformers import Qwen3Config

    from tah_amd.attention import build_attention_mask
    from tah_amd.cache import TaHDuoCache
    from tah_amd.hf_qwen3 import fused_attention_forward

    torch.manual_seed(seed)
    cfg = Qwen3Config(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=128, num_hidden_layers=1,
                      intermediate_size=512, vocab_size=128, rope_theta=1e6, attention_dropout=0.0)
    cfg._attn_implementation = "sdpa"
    layer = m.Qwen3Attention(cfg, layer_idx=0).to(device, torch.bfloat16).eval()
    with torch.no_grad():
        layer.q_norm.weight.copy_(1.0 + 0.1 * torch.randn(128))
        layer.k_norm.weight.copy_(1.0 + 0.1 * torch.randn(128))
    rope = m.Qwen3RotaryEmbedding(cfg).to(device)
    x = torch.randn(B, T, 256).to(torch.bfloat16).to(device)
    pos = torch.arange(T, device=device)[None].expand(B, T)
    valid = torch.ones(B, T, dtype=torch.long, device=device)
    with torch.no_grad():
        cos, sin = rope(x, pos)
        cache = TaHDuoCache()
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
        mask = build_attention_mask(pos, valid, cache, 0)
        dense = mask.dense(torch.bfloat16)
        want, _ = layer(x, (cos, sin), dense)                       # the module's own forward, no cache
        got, _ = fused_attention_forward(layer, x, (cos, sin), mask, past_key_values=cache)
    return got.float().cpu(), want.float().cpu()


def run_prefill_then_decode(device, B=2, T=20, steps=2, seed=1):
    """Prefill then decode steps of one layer: the module's own forward fed the reference's way (dense
    additive mask, cache returning the concatenated K/V) against the fused forward with slabs (decode kernel)."""
    m = pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    from transformers import Qwen3Config

    from tah_amd.attention import build_attention_mask
    from tah_amd.cache import TaHDuoCache
    from tah_amd.hf_qwen3 import fused_attention_forward

    torch.manual_seed(seed)
    cfg = Qwen3Config(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=128, num_hidden_layers=1,
                      intermediate_size=512, vocab_size=128, rope_theta=1e6, attention_dropout=0.0)
    cfg._attn_implementation = "sdpa"
    layer = m.Qwen3Attention(cfg, layer_idx=0).to(device, torch.bfloat16).eval()
    rope = m.Qwen3RotaryEmbedding(cfg).to(device)
    ref_cache, our_cache = TaHDuoCache(return_concat=True), TaHDuoCache().enable_slabs(T + steps + 2, 4)
    outs = []
    with torch.no_grad():
        for step in range(steps + 1):
            t = T if step == 0 else 1
            x = torch.randn(B, t, 256).to(torch.bfloat16).to(device)
            start = 0 if step == 0 else T + step - 1
            pos = (start + torch.arange(t, device=device))[None].expand(B, t).contiguous()
            valid = torch.ones(B, t, dtype=torch.long, device=device)
            cos, sin = rope(x, pos)
            res = []
            for cache, fused in ((ref_cache, False), (our_cache, True)):
                cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
                mask = build_attention_mask(pos, valid, cache, 0)
                if fused:
                    o, _ = fused_attention_forward(layer, x, (cos, sin), mask, past_key_values=cache)
                else:
                    o, _ = layer(x, (cos, sin), mask.dense(torch.bfloat16), past_key_values=cache)
                res.append(o.float().cpu())
            outs.append(res)
    return outs


def run_training_step(device, B=2, T=37, seed=3):
    """Forward and backward through one Qwen3Attention module, its own way (eager modules, SDPA, dense mask) and through
    the fused forward, from the same bf16 parameters: returns (output, gradient of the input, gradients of every
    parameter by name) for both."""
    m = pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    import copy

    from transformers import Qwen3Config

    from tah_amd.attention import build_attention_mask
    from tah_amd.cache import TaHDuoCache
    from tah_amd.hf_qwen3 import fused_attention_forward

    torch.manual_seed(seed)
    cfg = Qwen3Config(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=128, num_hidden_layers=1,
                      intermediate_size=512, vocab_size=128, rope_theta=1e6, attention_dropout=0.0)
    cfg._attn_implementation = "sdpa"
    layer = m.Qwen3Attention(cfg, layer_idx=0).to(device, torch.bfloat16).train()
    with torch.no_grad():
        layer.q_norm.weight.copy_(1.0 + 0.1 * torch.randn(128))
        layer.k_norm.weight.copy_(1.0 + 0.1 * torch.randn(128))
    fused = copy.deepcopy(layer)
    rope = m.Qwen3RotaryEmbedding(cfg).to(device)
    x0 = torch.randn(B, T, 256).to(torch.bfloat16).to(device)
    w = torch.randn(B, T, 256).to(torch.bfloat16).to(device)
    pos = torch.arange(T, device=device)[None].expand(B, T)
    valid = torch.ones(B, T, dtype=torch.long, device=device)
    with torch.no_grad():
        cos, sin = rope(x0, pos)
    out = []
    for mod, own in ((layer, True), (fused, False)):
        x = x0.clone().requires_grad_(True)
        cache = TaHDuoCache()
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
        mask = build_attention_mask(pos, valid, cache, 0)
        if own:
            y, _ = mod(x, (cos, sin), mask.dense(torch.bfloat16))
        else:
            y, _ = fused_attention_forward(mod, x, (cos, sin), mask, past_key_values=cache)
        (y.float() * w.float()).sum().backward()
        out.append((y.detach().float().cpu(), x.grad.float().cpu(), {n: p.grad.float().cpu() for n, p in mod.named_parameters()}))
    return out
