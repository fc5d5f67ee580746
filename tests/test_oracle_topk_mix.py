"""Pins oracle/topk_mix_ref.py (the restatement of tah_model.py:57-75) without the reference: torch's own
topk / softmax / sum in bf16, closed forms, and the tie rule on a hand-made row."""
import numpy as np
import torch

from oracle.topk_mix_ref import bf16_round, topk_indices, topk_mix
from tests.topk_mix_cases import make_case


def _torch_reference(logits, emb, k):
    """The reference's call sequence, verbatim in library routines, in bf16 on the CPU."""
    lg, em = torch.from_numpy(logits).to(torch.bfloat16), torch.from_numpy(emb).to(torch.bfloat16)
    kk = min(k, lg.shape[-1])
    tv, ti = torch.topk(lg, k=kk, dim=-1)
    pr = torch.softmax(tv, dim=-1)
    return torch.sum(pr.unsqueeze(-1) * em[ti], dim=-2).to(em.dtype).float().numpy()


def test_matches_torch_topk_softmax_sum_in_bf16_on_distinct_values():
    for seed, rows, V, H, k in ((0, 5, 700, 64, 100), (1, 3, 3000, 32, 17), (2, 2, 90, 16, 100)):
        logits, emb = make_case(seed, rows, V, H, distinct=True)
        got, want = topk_mix(logits, emb, k), _torch_reference(logits, emb, k)
        # same products and probabilities; only the float32 summation order differs: at most one bf16 step
        tol = np.maximum(np.abs(want), 1e-3) * 2.0 ** -7
        assert (np.abs(got - want) <= tol).all()
        assert (got == want).mean() > 0.9


def test_k1_is_the_argmax_row_and_selected_set_is_the_k_largest():
    logits, emb = make_case(3, 4, 500, 24, distinct=True)
    out = topk_mix(logits, emb, 1)
    assert np.array_equal(out, emb[np.argmax(logits, 1)])  # probability 1.0 times the row, exact in bf16
    idx = topk_indices(logits[0], 50)
    assert set(idx.tolist()) == set(np.argsort(logits[0])[-50:].tolist())
    assert (np.diff(logits[0][idx]) <= 0).all()


def test_constant_logits_take_the_lowest_indices_and_average_them():
    V, H, k = 300, 8, 100
    g = np.random.default_rng(5)
    emb = bf16_round(g.standard_normal((V, H)).astype(np.float32))
    logits = np.full((1, V), 1.5, dtype=np.float32)
    assert topk_indices(logits[0], k).tolist() == list(range(k))
    p = bf16_round(np.float32([1.0 / k]))[0]
    want = bf16_round(bf16_round(p * emb[:k]).sum(0, dtype=np.float32))
    assert np.array_equal(topk_mix(logits, emb, k)[0], want)
    # k >= V: every row takes part
    p = bf16_round(np.float32([1.0 / V]))[0]
    want = bf16_round(bf16_round(p * emb).sum(0, dtype=np.float32))
    assert np.array_equal(topk_mix(logits, emb, 1000)[0], want)


def test_ties_at_the_kth_place_go_to_the_lower_index():
    row = np.float32([0.0, 2.0, 1.0, 1.0, 3.0, 1.0, -1.0])
    assert topk_indices(row, 3).tolist() == [4, 1, 2]
    assert topk_indices(row, 4).tolist() == [4, 1, 2, 3]
    assert topk_indices(row, 5).tolist() == [4, 1, 2, 3, 5]
