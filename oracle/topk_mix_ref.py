"""CPU restatement of the reference's soft input update for hard tokens.  TEST INFRASTRUCTURE: only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg may import this package.

Follows ``topk_softmax_input_update`` (tah/model/tah_model.py:57-75): ``torch.topk(logits, k)``, softmax over the
k values, gather of the k embedding rows, probability-weighted sum, result in the embedding's dtype -- evaluated
the way bf16 eager arithmetic evaluates it: softmax in float32 rounded to bf16, each product rounded to bf16,
the sum accumulated in float32 and rounded once.  Where ``torch.topk`` leaves the choice among equal values at
the k-th place open, the lower vocabulary indices are taken.

Pinned in tests/test_oracle_topk_mix.py against torch's own ``topk`` / ``softmax`` / ``sum`` in bf16 on inputs
whose values are all distinct, and against closed forms (k = 1: the arg-max row; constant logits with k = V: the
rounded mean of rounded rows; tie-breaking by index on a hand-made row).
"""
from __future__ import annotations

import numpy as np


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even), returned as float32."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = ((b >> 16) & 1) + np.uint32(0x7FFF)
    return ((b + r) & np.uint32(0xFFFF0000)).view(np.float32)


def topk_indices(row: np.ndarray, k: int) -> np.ndarray:
    """Indices of the k largest values, larger values first, lower index first among equal values."""
    order = np.argsort(-row.astype(np.float64), kind="stable")
    return order[:k]


def topk_mix(logits: np.ndarray, embedding: np.ndarray, topk: int) -> np.ndarray:
    """logits [rows, V], embedding [V, H]: float32 arrays holding bf16-representable values -> float32 [rows, H]."""
    rows, V = logits.shape
    k = min(topk, V)
    out = np.zeros((rows, embedding.shape[1]), dtype=np.float32)
    for r in range(rows):
        idx = np.sort(topk_indices(logits[r], k))  # summation order: by index
        v = logits[r, idx].astype(np.float32)
        e = np.exp(v - v.max(), dtype=np.float32)
        p = bf16_round(e / e.sum(dtype=np.float32))
        prod = bf16_round(p[:, None] * embedding[idx].astype(np.float32))
        out[r] = bf16_round(prod.sum(0, dtype=np.float32))
    return out
