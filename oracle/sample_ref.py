"""CPU restatement of the reference's token sampler.  TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg may import this package.

Follows ``sample_next_token`` (tah/model/utils.py:84-125) for ``do_sample=True`` and ``top_k == 0``:
``softmax(logits / temperature)``; with ``min_p > 0`` the tokens whose probability is below ``min_p`` times the largest
one are dropped and the rest renormalised (utils.py:105-108); with ``top_p < 1`` the tokens are put in descending
order, a token is dropped when the cumulative probability up to and including its predecessor exceeds ``top_p`` (the
shift of utils.py:118-119 keeps the token that crosses), and the rest renormalised (utils.py:115-123).  Evaluated in
float64.  ``torch.sort`` leaves the order of equal probabilities open; here the lower vocabulary index comes first (a
stable sort).  The reference then draws with ``torch.multinomial`` (utils.py:125), i.e. from exactly this
distribution with torch's generator; ``draw`` below is the inverse-CDF draw from the same distribution for a given
uniform number, over the tokens in the order of the sort: the first token at which the cumulative kept probability
exceeds u.

Pinned in tests/test_oracle_sample.py: against torch's own ``softmax`` / ``sort`` / ``cumsum`` / ``scatter`` pipeline in
float64 on rows without ties; against brute force over all subsets on tiny rows (top_p keeps the smallest prefix of
the descending order whose mass exceeds top_p, or everything); closed forms (constant rows: top_p keeps
floor(top_p * V) + 1 tokens, the lowest indices; min_p on a two-level row); and ``draw`` against exhaustive
frequencies on a grid of u.
"""
from __future__ import annotations

import numpy as np


def final_logits(logits: np.ndarray, prev: np.ndarray | None = None, add_prev: np.ndarray | None = None) -> np.ndarray:
    """Rows whose ``add_prev`` entry is not 0: ``prev + logits`` rounded to bf16 (float32 arrays of bf16 values)."""
    from oracle.topk_mix_ref import bf16_round
    out = np.array(logits, dtype=np.float32)
    if prev is not None and add_prev is not None:
        sel = np.asarray(add_prev) != 0
        out[sel] = bf16_round(prev[sel].astype(np.float32) + logits[sel].astype(np.float32))
    return out


def filtered_probs(logits: np.ndarray, temperature: float, top_p: float = 1.0, min_p: float = 0.0) -> np.ndarray:
    """[rows, V] -> float64 [rows, V]: the distribution the reference draws from, zero outside the filters."""
    x = np.asarray(logits, dtype=np.float64) / float(temperature)
    x = x - x.max(axis=-1, keepdims=True)
    p = np.exp(x)
    p /= p.sum(axis=-1, keepdims=True)
    if min_p > 0.0:
        p = np.where(p >= min_p * p.max(axis=-1, keepdims=True), p, 0.0)
        p /= p.sum(axis=-1, keepdims=True)
    if top_p < 1.0:
        for r in range(p.shape[0]):
            order = np.argsort(-p[r], kind="stable")
            cum = np.cumsum(p[r, order])
            remove = np.zeros(order.size, dtype=bool)
            remove[1:] = cum[:-1] > top_p
            p[r, order[remove]] = 0.0
        p /= p.sum(axis=-1, keepdims=True)
    return p


def draw(probs: np.ndarray, u: np.ndarray) -> np.ndarray:
    """The token of each row at which the cumulative probability, over the tokens in descending order (equal ones by
    ascending index), first exceeds ``u`` (one number in [0, 1) per row)."""
    out = np.zeros(probs.shape[0], dtype=np.int64)
    for r in range(probs.shape[0]):
        order = np.argsort(-probs[r], kind="stable")
        cum = np.cumsum(probs[r, order])
        kept = int((probs[r] > 0).sum())
        i = int(np.searchsorted(cum[:kept], u[r] * cum[kept - 1], side="right"))
        out[r] = order[min(i, kept - 1)]
    return out


def draw_interval(probs: np.ndarray, token: np.ndarray):
    """For each row the interval [lo, hi) of u for which ``draw`` returns ``token`` (as fractions of the kept mass)."""
    lo = np.zeros(probs.shape[0])
    hi = np.zeros(probs.shape[0])
    for r in range(probs.shape[0]):
        order = np.argsort(-probs[r], kind="stable")
        cum = np.cumsum(probs[r, order])
        where = int(np.nonzero(order == token[r])[0][0])
        lo[r] = (cum[where - 1] if where else 0.0) / cum[-1]
        hi[r] = cum[where] / cum[-1]
    return lo, hi
