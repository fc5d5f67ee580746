"""tah_sample_rows (temperature / min_p / top_p sampling without a sort, tah/model/utils.py:84-125 with top_k == 0)
against its oracle: on the CPU execution build of the kernel, and on the GPU through the C ABI.

Tolerances.  The kernel sums in float32 and takes exp through the hardware's exp2; the oracle is float64.
Probabilities of kept tokens agree to 3e-5 relative.  The kept set must be the oracle's, except for tokens at the very
edge of a filter: a token may differ when the mass before it is within 2e-6 of top_p (relative to the total) or its
probability within 2e-5 relative of min_p times the largest (none of the seeded cases below has such a token; the
check reports them if a change of seed produces one).  A drawn token is right when the caller's u lies in the
token's interval of the oracle's cumulative distribution, widened by 1e-5."""
import numpy as np
import pytest
import torch

from oracle import sample_ref as S
from oracle.topk_mix_ref import bf16_round
from tests import emu_util


def make_rows(seed, rows, V, style):
    rng = np.random.default_rng(seed)
    if style == "peaked":      # a language model's shape: a few tokens carry the mass
        x = rng.standard_normal((rows, V)) * 3.0
    elif style == "flat":      # random weights: every token matters, the top_p cut lies deep in the row
        x = rng.standard_normal((rows, V)) * 0.05 + 0.3
    elif style == "negative":  # no positive logit: the largest key lies in the lower half of the key space
        x = -np.abs(rng.standard_normal((rows, V))) * 4.0 - 1.0
    elif style == "ties":      # few distinct values: every filter cuts through a group of equal tokens
        x = rng.integers(-6, 3, size=(rows, V)).astype(np.float64) * 0.5
    elif style == "wide":      # values across both halves of the key space, with -inf entries (masked tokens)
        x = rng.standard_normal((rows, V)) * 8.0
        x[:, ::7] = -np.inf
    else:
        raise ValueError(style)
    return bf16_round(x.astype(np.float32))


def check_probs(got, want, top_p, min_p):
    got = got.astype(np.float64)
    for r in range(want.shape[0]):
        a, b = got[r] > 0, want[r] > 0
        diff = np.nonzero(a != b)[0]
        assert diff.size == 0, f"row {r}: kept sets differ at tokens {diff[:8].tolist()} ({diff.size}); kept {int(a.sum())} vs {int(b.sum())}"
        np.testing.assert_allclose(got[r][b], want[r][b], rtol=3e-5, atol=0)
        assert abs(got[r].sum() - 1.0) < 1e-4


def check_tokens(tok, u, want_probs):
    lo, hi = S.draw_interval(want_probs, tok)
    for r in range(len(tok)):
        assert want_probs[r, tok[r]] > 0, f"row {r}: token {tok[r]} is outside the filters"
        assert lo[r] - 1e-5 <= u[r] < hi[r] + 1e-5, f"row {r}: u={u[r]} token {tok[r]} interval [{lo[r]}, {hi[r]})"


def run_case(device, seed, rows, V, style, temperature, top_p, min_p, with_prev=False):
    from tah_amd import ops
    x = make_rows(seed, rows, V, style)
    rng = np.random.default_rng(seed + 100)
    u = rng.random(rows).astype(np.float32)
    u[0] = 0.0
    if rows > 1:
        u[1] = np.float32(1.0 - 2.0 ** -24)
    kw = {}
    final = x
    if with_prev:
        prev = bf16_round((rng.standard_normal((rows, V)) * 0.7).astype(np.float32))
        add = (np.arange(rows) % 2).astype(np.int32)
        final = S.final_logits(x, prev, add)
        kw = dict(logits_prev=torch.from_numpy(prev).to(torch.bfloat16).to(device), add_prev=torch.from_numpy(add).to(device))
    want = S.filtered_probs(final, temperature, top_p, min_p)
    lt = torch.from_numpy(x).to(torch.bfloat16).to(device)
    got = ops.sample_probs(lt, temperature, top_p=top_p, min_p=min_p, **kw)
    check_probs(got.cpu().numpy(), want, top_p, min_p)
    tok = ops.sample_rows(lt, torch.from_numpy(u).to(device), temperature, top_p=top_p, min_p=min_p, **kw)
    check_tokens(tok.cpu().numpy(), u, want)
    return want


EMU_CASES = [
    (0, 2, 1500, "peaked", 0.6, 0.95, 0.0, False),
    (1, 2, 1500, "flat", 1.0, 0.9, 0.0, False),
    (2, 1, 9003, "ties", 0.7, 0.8, 0.0, False),       # odd length: the last piece is ragged
    (3, 2, 3000, "negative", 1.0, 0.5, 0.05, False),
    (4, 2, 4000, "wide", 0.8, 0.97, 0.0, True),
    (5, 1, 700, "ties", 1.0, 1.0, 0.3, False),        # min_p alone, cutting between two levels
    (6, 2, 900, "peaked", 1.3, 1.0, 0.0, True),       # plain temperature sampling
    (7, 1, 17000, "flat", 0.6, 0.3, 0.0, False),
]


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
@pytest.mark.parametrize("seed,rows,V,style,temperature,top_p,min_p,with_prev", EMU_CASES)
def test_sample_rows_on_cpu_shim(seed, rows, V, style, temperature, top_p, min_p, with_prev):
    with emu_util.emulated():
        run_case("cpu", seed, rows, V, style, temperature, top_p, min_p, with_prev)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_sample_rows_row_enable_and_refusals_on_cpu_shim():
    from tah_amd import ops
    from tah_amd._capi import TahDuoError
    x = torch.from_numpy(make_rows(9, 3, 800, "peaked")).to(torch.bfloat16)
    u = torch.tensor([0.3, 0.6, 0.9])
    with emu_util.emulated():
        out = torch.full((3,), -5, dtype=torch.int64)
        ops.sample_rows(x, u, 0.7, top_p=0.9, row_enable=torch.tensor([1, 0, 1], dtype=torch.uint8), out=out)
        full = ops.sample_rows(x, u, 0.7, top_p=0.9)
        for bad in (dict(temperature=0.0), dict(temperature=0.7, top_p=0.0), dict(temperature=0.7, min_p=1.5)):
            with pytest.raises(TahDuoError):
                ops.sample_rows(x, u, bad.pop("temperature"), **bad)
    assert out[1] == -5 and out[0] == full[0] and out[2] == full[2]


GPU_CASES = [
    (20, 4, 151936, "peaked", 0.6, 0.95, 0.0, False),
    (21, 4, 151936, "flat", 0.6, 0.95, 0.0, True),
    (22, 3, 151936, "ties", 1.0, 0.9, 0.0, False),
    (23, 3, 151936, "wide", 0.7, 0.99, 0.02, True),
    (24, 2, 151936, "negative", 1.0, 1.0, 0.1, False),
    (25, 5, 32000, "peaked", 1.0, 0.5, 0.0, False),
    (26, 2, 155648, "flat", 1.5, 1.0, 0.0, False),
    (27, 3, 50257, "peaked", 0.8, 0.9, 0.05, False),
]


@pytest.mark.gpu
@pytest.mark.parametrize("seed,rows,V,style,temperature,top_p,min_p,with_prev", GPU_CASES)
def test_sample_rows_gpu(seed, rows, V, style, temperature, top_p, min_p, with_prev):
    run_case("cuda", seed, rows, V, style, temperature, top_p, min_p, with_prev)


@pytest.mark.gpu
@pytest.mark.parametrize("style,temperature,top_p,min_p", [("peaked", 0.6, 0.95, 0.0), ("flat", 0.6, 0.95, 0.0), ("peaked", 1.0, 0.8, 0.05),
                                                          ("wide", 0.7, 1.0, 0.01)])
def test_sample_rows_gpu_against_the_engines_torch_sampler(style, temperature, top_p, min_p):
    """The kept set and the renormalised probabilities are those of ``TaHDecodeEngine.filtered_probs`` (the torch
    restatement of the reference's sampler that the engine used for this case: a float32 sort over the vocabulary)."""
    from tah_amd import ops
    from tah_amd.engine import TaHDecodeEngine
    x = torch.from_numpy(make_rows(31, 6, 151936, style)).to(torch.bfloat16).cuda()
    want = TaHDecodeEngine.filtered_probs(x.float(), temperature, top_p=top_p, min_p=min_p)
    got = ops.sample_probs(x, temperature, top_p=top_p, min_p=min_p)
    kept_w, kept_g = want > 0, got > 0
    # float32 against float32, summed in different orders: a token may flip at the very edge of top_p
    flips = (kept_w != kept_g).sum(dim=-1)
    assert int(flips.max()) <= 1, flips.tolist()
    both = kept_w & kept_g
    rel = ((got - want).abs() / want.clamp_min(1e-30))[both]
    assert float(rel.max()) < (1e-3 if int(flips.max()) else 1e-4), float(rel.max())


@pytest.mark.gpu
def test_sample_rows_gpu_draw_frequencies():
    """Many draws from one row: the frequencies are the filtered distribution's (each within five standard deviations)."""
    from tah_amd import ops
    V, n = 64, 200000
    row = make_rows(41, 1, V, "peaked")
    want = S.filtered_probs(row, 0.9, 0.9, 0.0)[0]
    x = torch.from_numpy(row).to(torch.bfloat16).cuda().expand(n, V).contiguous()
    g = torch.Generator(device="cuda").manual_seed(5)
    tok = ops.sample_rows(x, torch.rand(n, device="cuda", generator=g), 0.9, top_p=0.9)
    freq = torch.bincount(tok, minlength=V).double().cpu().numpy() / n
    sd = np.sqrt(np.maximum(want * (1 - want), 1e-12) / n)
    assert (freq[want == 0] == 0).all()
    assert (np.abs(freq - want) <= 5 * sd + 1e-9).all(), float((np.abs(freq - want) / sd).max())
