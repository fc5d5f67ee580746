"""Attention-layer forward for Hugging Face ``Qwen3Attention`` modules built on this library's kernels.

``Qwen3Attention.forward`` (third party: transformers/models/qwen3/modeling_qwen3.py, the layer the
reference's base model runs, tah/model/tah_model.py:616-623) does, between the projections and the
output projection: ``q_norm`` / ``k_norm`` per head, ``apply_rotary_pos_emb``, ``past_key_values.update``
and the attention-interface call.  :func:`fused_attention_forward` is that method with the norm and
rotary steps replaced by one ``tah_qk_prep`` launch on the token-major projections and the attention
call bound to :func:`tah_amd.attention.duo_attention_forward`.  Differentiable: under autograd the
preparation runs as ``tah_qk_prep`` / ``tah_qk_prep_bwd`` and the attention as the varlen forward / backward
kernels.  Use::

    from tah_amd.hf_qwen3 import patch_attention_layers
    patch_attention_layers(model)          # every Qwen3Attention in the model
"""
from __future__ import annotations

import types
from typing import Optional, Tuple

import torch

from .attention import duo_attention_forward
from .kv_cache import qk_norm_rope


def fused_attention_forward(self, hidden_states: torch.Tensor, position_embeddings: Tuple[torch.Tensor, torch.Tensor],
                            attention_mask, past_key_values=None, past_key_value=None, cache_position=None,
                            **kwargs) -> Tuple[torch.Tensor, None]:
    """Same arguments and result as ``Qwen3Attention.forward`` (``past_key_value`` is the keyword of
    transformers 4.x, ``past_key_values`` of 5.x).  ``attention_mask`` is what
    :func:`tah_amd.attention.build_attention_mask` returned (or the reference's dense additive mask)."""
    del cache_position, kwargs
    cache = past_key_values if past_key_values is not None else past_key_value
    B, T = hidden_states.shape[:2]
    D = self.head_dim
    q = self.q_proj(hidden_states).view(B * T, -1, D)
    k = self.k_proj(hidden_states).view(B * T, -1, D)
    v = self.v_proj(hidden_states).view(B, T, -1, D)
    cos, sin = position_embeddings
    if cos.shape[0] != B:  # (1, T, D) tables shared by the batch
        cos, sin = cos.expand(B, T, D), sin.expand(B, T, D)
    eps = getattr(self.q_norm, "variance_epsilon", getattr(self.q_norm, "eps", 1e-6))
    q, k = qk_norm_rope(q, k, self.q_norm.weight, self.k_norm.weight, cos.reshape(B * T, D), sin.reshape(B * T, D), eps)
    query_states = q.view(B, T, -1, D).transpose(1, 2)
    key_states = k.view(B, T, -1, D).transpose(1, 2)
    value_states = v.transpose(1, 2)
    if cache is not None:
        key_states, value_states = cache.update(key_states, value_states, self.layer_idx)
    attn_output, _ = duo_attention_forward(self, query_states, key_states, value_states, attention_mask, dropout=0.0,
                                           scaling=self.scaling)
    return self.o_proj(attn_output.reshape(B, T, -1).contiguous()), None


def patch_attention_layers(model: torch.nn.Module) -> int:
    """Bind :func:`fused_attention_forward` to every ``Qwen3Attention`` module of ``model``; returns how many."""
    n = 0
    for m in model.modules():
        if type(m).__name__ == "Qwen3Attention":
            m.forward = types.MethodType(fused_attention_forward, m)
            n += 1
    return n
