"""CPU restatement of the reference's learned iteration decider.  TEST INFRASTRUCTURE: only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package.

Follows ``MLPIterDecider.forward`` (tah/model/iter_decider.py:265-301) with its helpers ``_select_hidden_features``
(:244-263), ``_ClassifierBlock.forward`` (:128) and ``_ClassifierBackbone.forward`` (:182-186), in float64 numpy on a
dict of arrays keyed like the module's state dict: the k largest logits, largest first; the selected layers of the
hidden states side by side; optional LayerNorm of those and softmax of the logit values; logits_projection;
combined_projection over [hidden features | projected logit values]; backbone = input_projection, residual blocks
``dim_change(x) + W2 gelu(W1 LayerNorm(x))`` (erf GELU, LayerNorm eps 1e-5, dropout inactive), final LayerNorm and a
projection to one logit; sigmoid(logit) > threshold; past the iteration cap nobody continues and the logit is -10.

Pinned in tests/test_oracle_decider.py: against the same network assembled from torch's own ``nn.Linear`` /
``nn.LayerNorm`` / ``nn.GELU`` / ``torch.topk`` modules in float64 (block widths, residual wiring, order of the
concatenation, descending order of the logit values each checked by a case that a mistake there fails), and closed
forms (all-zero weights: the output bias; the cap: all False and -10).
"""
from __future__ import annotations

import math

import numpy as np

STOP_LOGIT = -10.0


def _lin(p, name, x):
    return x @ p[name + ".weight"].astype(np.float64).T + p[name + ".bias"].astype(np.float64)


def _layer_norm(p, name, x, eps=1e-5):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * p[name + ".weight"].astype(np.float64) + p[name + ".bias"].astype(np.float64)


_erf = np.vectorize(math.erf)


def _gelu(x):
    return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))


def topk_values(logits: np.ndarray, k: int) -> np.ndarray:
    """The k largest entries of every row, largest first (iter_decider.py:281)."""
    return -np.sort(-logits.astype(np.float64), axis=-1)[..., : min(k, logits.shape[-1])]


def hidden_features(all_hidden_states, layer_nums, lead, hidden_size):
    """iter_decider.py:244-263"""
    slots = max(1, len(layer_nums))
    if all_hidden_states is None:
        return np.zeros((*lead, hidden_size * slots))
    hs = np.asarray(all_hidden_states, dtype=np.float64)
    if hs.ndim == len(lead) + 1:
        hs = hs[..., None, :]
    pick = list(layer_nums) or [hs.shape[-2] - 1]
    return np.take(hs, pick, axis=-2).reshape(*lead, hidden_size * slots)


def backbone(p, x, n_blocks):
    """iter_decider.py:182-186 with the block of :128"""
    x = _lin(p, "backbone.input_projection", x)
    for i in range(n_blocks):
        b = f"backbone.blocks.{i}"
        y = _lin(p, b + ".mlp.3", _gelu(_lin(p, b + ".mlp.0", _layer_norm(p, b + ".layer_norm", x))))
        x = (_lin(p, b + ".dim_change", x) if b + ".dim_change.weight" in p else x) + y
    return _lin(p, "backbone.output_layer.1", _layer_norm(p, "backbone.output_layer.0", x))


def decide(p, logits, iter_depth, all_hidden_states=None, *, topk=100, hidden_size=1024, layer_nums=(16, 20, 24, 28),
           n_blocks=3, normalize_input=False, max_iter=3):
    """(decision, decision_logits) of iter_decider.py:265-301; ``p``: state-dict names -> arrays."""
    lead = logits.shape[:-1]
    if iter_depth >= max_iter:
        return np.zeros(lead, dtype=bool), np.full(lead, STOP_LOGIT)
    feats = hidden_features(all_hidden_states, layer_nums, lead, hidden_size)
    top = topk_values(logits, topk)
    if normalize_input:
        feats = _layer_norm(p, "layer_norm_hidden_states", feats)
        e = np.exp(top - top.max(-1, keepdims=True))
        top = e / e.sum(-1, keepdims=True)
    x = _lin(p, "combined_projection", np.concatenate([feats, _lin(p, "logits_projection", top)], axis=-1))
    z = backbone(p, x, n_blocks)[..., 0]
    return 1.0 / (1.0 + np.exp(-z)) > float(p["threshold"]), z
