"""A tiny transformers Qwen3Model stepped the way the reference's forward loop steps its base model
(tah/model/tah_model.py:604-623: stage depth / positions / valid flags on the cache, build the mask, call the
model with the 4-D mask and the cache), once with the reference's ingredients (SDPA, dense additive mask, cache
that returns the concatenated K/V) and once with this library's (DuoMask, fused attention layers)."""
import copy

import pytest
import torch


def run(device, B=2, T=24, layers=2, p_hard=0.3, seed=0):
    pytest.importorskip("transformers.models.qwen3.modeling_qwen3")
    from transformers import Qwen3Config, Qwen3Model

    from tah_amd.attention import build_attention_mask
    from tah_amd.cache import TaHDuoCache
    from tah_amd.hf_qwen3 import patch_attention_layers
    from tah_amd.pack import gather_active

    torch.manual_seed(seed)
    cfg = Qwen3Config(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
                      num_hidden_layers=layers, intermediate_size=512, vocab_size=128, rope_theta=1e6,
                      attention_dropout=0.0)
    cfg._attn_implementation = "sdpa"
    ref_model = Qwen3Model(cfg).to(device, torch.bfloat16).eval()
    our_model = copy.deepcopy(ref_model)
    assert patch_attention_layers(our_model) == layers

    embeds = torch.randn(B, T, 256).to(torch.bfloat16).to(device)
    pos = torch.arange(T, device=device)[None].expand(B, T).contiguous()
    valid = torch.ones(B, T, dtype=torch.long, device=device)
    hard = torch.rand(B, T, device=device) < p_hard
    hard[:, 0] = True  # every row has at least one hard token
    outs = []
    with torch.no_grad():
        for model, cache, ours in ((ref_model, TaHDuoCache(return_concat=True), False), (our_model, TaHDuoCache(), True)):
            res = []
            # depth 0: every token
            x, p, v = embeds, pos, valid
            for depth in (0, 1):
                if depth == 1:  # depth 1: the hard tokens only, packed to the left (tah_model.py:589-593)
                    pad_mask, x, p, v = gather_active(hard, embeds * 0.5 + 0.25, pos, valid)
                    v = v * (~pad_mask).long()
                cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = depth, p, v
                mask = build_attention_mask(p, v, cache, depth)
                mask_arg = {"full_attention": mask if ours else mask.dense(torch.bfloat16)}
                out = model(inputs_embeds=x, attention_mask=mask_arg, position_ids=p, past_key_values=cache,
                            use_cache=True).last_hidden_state
                keep = v.bool()
                res.append((out.float() * keep[..., None]).cpu())
            outs.append(res)
    return outs
