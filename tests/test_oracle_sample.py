"""Pins oracle/sample_ref.py (the restatement of sample_next_token, tah/model/utils.py:84-125, top_k == 0) against torch's
own routines, brute force on tiny rows and closed forms.  No GPU."""
import itertools

import numpy as np
import pytest
import torch

from oracle import sample_ref as S


def torch_pipeline(logits, temperature, top_p, min_p):
    """The same filters composed from torch's library routines in float64 (softmax, sort, cumsum, scatter)."""
    probs = torch.softmax(torch.from_numpy(logits).double() / temperature, dim=-1)
    if min_p > 0.0:
        probs = torch.where(probs >= min_p * probs.max(dim=-1, keepdim=True).values, probs, torch.zeros_like(probs))
        probs = probs / probs.sum(dim=-1, keepdim=True)
    if top_p < 1.0:
        sp, si = torch.sort(probs, descending=True, dim=-1, stable=True)
        remove = torch.cumsum(sp, dim=-1) > top_p
        remove = torch.cat([torch.zeros_like(remove[..., :1]), remove[..., :-1]], dim=-1)
        probs = torch.where(torch.zeros_like(remove).scatter_(-1, si, remove), torch.zeros_like(probs), probs)
        probs = probs / probs.sum(dim=-1, keepdim=True)
    return probs.numpy()


@pytest.mark.parametrize("temperature,top_p,min_p", [(1.0, 1.0, 0.0), (0.6, 0.95, 0.0), (0.8, 1.0, 0.05), (1.3, 0.7, 0.02), (0.5, 0.2, 0.0)])
def test_against_torch_routines_on_rows_without_ties(temperature, top_p, min_p):
    rng = np.random.default_rng(7)
    logits = (rng.standard_normal((5, 3000)) * 3.0).astype(np.float32)
    got = S.filtered_probs(logits, temperature, top_p, min_p)
    want = torch_pipeline(logits, temperature, top_p, min_p)
    assert np.array_equal(got > 0, want > 0)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=0)
    np.testing.assert_allclose(got.sum(-1), 1.0, rtol=1e-12)


def test_top_p_keeps_the_smallest_set_of_largest_tokens_whose_mass_exceeds_it_brute_force():
    rng = np.random.default_rng(11)
    for trial in range(40):
        V = int(rng.integers(2, 8))
        logits = rng.standard_normal((1, V)).astype(np.float32) * 2
        top_p = float(rng.uniform(0.05, 0.99))
        p = np.exp(logits[0].astype(np.float64))
        p /= p.sum()
        best = None  # smallest subset size whose best subset has mass > top_p; all tokens if none does
        for n in range(1, V + 1):
            m, sub = max((sum(p[list(c)]), c) for c in itertools.combinations(range(V), n))
            if m > top_p:
                best = set(sub)
                break
        if best is None:
            best = set(range(V))
        got = S.filtered_probs(logits, 1.0, top_p, 0.0)[0]
        assert set(np.nonzero(got)[0].tolist()) == best, (trial, p, top_p)
        np.testing.assert_allclose(got[sorted(best)], p[sorted(best)] / p[sorted(best)].sum(), rtol=1e-12)


def test_closed_forms():
    # constant row: all probabilities 1/V; the token after which the running sum exceeds top_p is the last one kept,
    # equal tokens in index order
    for V, top_p in ((10, 0.35), (64, 0.5001), (7, 0.999), (5, 0.01)):
        got = S.filtered_probs(np.zeros((1, V), np.float32), 0.7, top_p, 0.0)[0]
        n = min(V, int(np.floor(top_p * V + 1e-9)) + 1)
        assert np.nonzero(got)[0].tolist() == list(range(n)), (V, top_p)
        np.testing.assert_allclose(got[:n], 1.0 / n, rtol=1e-12)
    # two levels: three tokens at a, five at a - T ln 4, i.e. a quarter of the largest probability each
    T = 0.6
    row = np.array([[2.0] * 3 + [2.0 - T * np.log(4.0)] * 5], dtype=np.float64)
    keep_all = S.filtered_probs(row, T, 1.0, 0.2)[0]
    np.testing.assert_allclose(keep_all, np.array([4.0] * 3 + [1.0] * 5) / 17.0, rtol=1e-12)
    only_top = S.filtered_probs(row, T, 1.0, 0.3)[0]
    np.testing.assert_allclose(only_top, np.array([1 / 3.0] * 3 + [0.0] * 5), rtol=1e-12)
    # both filters: min_p first (three tokens of 1/3 left), then top_p = 0.5: two tokens
    both = S.filtered_probs(row, T, 0.5, 0.3)[0]
    np.testing.assert_allclose(both, np.array([0.5, 0.5] + [0.0] * 6), rtol=1e-12)


def test_draw_is_the_inverse_cdf_over_the_sorted_order():
    probs = np.array([[0.1, 0.4, 0.0, 0.4, 0.1]])
    # order: 1, 3 (equal, lower index first), 0, 4; intervals [0, .4) [.4, .8) [.8, .9) [.9, 1)
    for u, tok in ((0.0, 1), (0.39, 1), (0.4, 3), (0.79, 3), (0.8, 0), (0.95, 4), (0.999999, 4)):
        assert S.draw(probs, np.array([u]))[0] == tok, u
    lo, hi = S.draw_interval(probs, np.array([0]))
    assert abs(lo[0] - 0.8) < 1e-12 and abs(hi[0] - 0.9) < 1e-12
    rng = np.random.default_rng(3)
    p = rng.dirichlet(np.ones(12))[None]
    N = 20000
    toks = np.concatenate([S.draw(p, np.array([(i + 0.5) / N])) for i in range(N)])
    freq = np.bincount(toks, minlength=12) / N
    assert np.abs(freq - p[0]).max() <= 1.0 / N + 1e-12


def test_final_logits_adds_in_bf16_where_asked():
    from oracle.topk_mix_ref import bf16_round
    rng = np.random.default_rng(5)
    a = bf16_round(rng.standard_normal((3, 50)).astype(np.float32))
    b = bf16_round(rng.standard_normal((3, 50)).astype(np.float32))
    got = S.final_logits(a, b, np.array([0, 1, 0]))
    want = (torch.from_numpy(b[1]).bfloat16() + torch.from_numpy(a[1]).bfloat16()).float().numpy()
    assert np.array_equal(got[1], want) and np.array_equal(got[0], a[0]) and np.array_equal(got[2], a[2])
