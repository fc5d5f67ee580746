"""Pins oracle/decider_ref.py (the float64 restatement of MLPIterDecider.forward, tah/model/iter_decider.py:193-301)
without the reference: every primitive against torch's own routine, and the wiring by cases a mistake there fails."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import decider_ref as R

rng = np.random.default_rng(0)


def _params(hidden=8, slots=2, k=5, dims=(6, 10, 6), ex=2):
    """Random float64 parameters under the reference's state-dict names, block widths as iter_decider.py:168-172
    lays them out: dims[i] -> dims[i + 1], then the last width once more."""
    p = {"threshold": np.array(0.5)}
    def lin(name, i, o):
        p[name + ".weight"], p[name + ".bias"] = rng.standard_normal((o, i)) * 0.5, rng.standard_normal(o) * 0.3
    def ln(name, n):
        p[name + ".weight"], p[name + ".bias"] = 1 + rng.standard_normal(n) * 0.2, rng.standard_normal(n) * 0.2
    ln("layer_norm_hidden_states", hidden * slots)
    lin("logits_projection", k, hidden)
    lin("combined_projection", hidden * slots + hidden, dims[0])
    lin("backbone.input_projection", dims[0], dims[0])
    widths = list(dims) + [dims[-1]]
    for i, (a, b) in enumerate(zip(widths[:-1], widths[1:])):
        ln(f"backbone.blocks.{i}.layer_norm", a)
        lin(f"backbone.blocks.{i}.mlp.0", a, a * ex)
        lin(f"backbone.blocks.{i}.mlp.3", a * ex, b)
        if a != b:
            lin(f"backbone.blocks.{i}.dim_change", a, b)
    ln("backbone.output_layer.0", dims[-1])
    lin("backbone.output_layer.1", dims[-1], 1)
    return p


def _torch_decide(p, logits, hs, k, layer_nums, n_blocks, normalize):
    """The same network from torch's own routines, float64."""
    t = {n: torch.from_numpy(np.asarray(v, dtype=np.float64)) for n, v in p.items()}
    lin = lambda n, x: F.linear(x, t[n + ".weight"], t[n + ".bias"])
    ln = lambda n, x: F.layer_norm(x, x.shape[-1:], t[n + ".weight"], t[n + ".bias"], 1e-5)
    feats = torch.index_select(hs, -2, torch.tensor(layer_nums)).flatten(-2)
    top = torch.topk(logits, k, dim=-1).values
    if normalize:
        feats, top = ln("layer_norm_hidden_states", feats), torch.softmax(top, -1)
    x = lin("combined_projection", torch.cat([feats, lin("logits_projection", top)], -1))
    x = lin("backbone.input_projection", x)
    for i in range(n_blocks):
        b = f"backbone.blocks.{i}"
        skip = lin(b + ".dim_change", x) if b + ".dim_change.weight" in t else x
        x = skip + lin(b + ".mlp.3", F.gelu(lin(b + ".mlp.0", ln(b + ".layer_norm", x))))
    z = lin("backbone.output_layer.1", ln("backbone.output_layer.0", x)).squeeze(-1)
    return torch.sigmoid(z) > 0.5, z


def _case(normalize):
    p = _params()
    logits = rng.standard_normal((2, 3, 40)) * 3
    hs = rng.standard_normal((2, 3, 4, 8))
    dec, z = R.decide(p, logits, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3, normalize_input=normalize)
    tdec, tz = _torch_decide(p, torch.from_numpy(logits), torch.from_numpy(hs), 5, [1, 3], 3, normalize)
    assert np.allclose(z, tz.numpy(), rtol=1e-10, atol=1e-10) and (dec == tdec.numpy()).all()
    return p, logits, hs, z


def test_against_torch_routines():
    _case(False)
    _case(True)


def test_logit_values_enter_largest_first_and_after_the_hidden_features():
    p, logits, hs, z = _case(False)
    # only logit slot 0 feeds the network: nothing but each token's largest logit may matter
    q = dict(p)
    w = np.zeros_like(p["logits_projection.weight"]); w[:, 0] = p["logits_projection.weight"][:, 0]
    q["logits_projection.weight"] = w
    shuffled = np.take_along_axis(logits, rng.permuted(np.tile(np.arange(40), (2, 3, 1)), axis=-1), -1)
    lower = np.where(logits == logits.max(-1, keepdims=True), logits, logits - 5.0)   # everything but the maximum moved
    za = R.decide(q, logits, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1]
    assert np.allclose(za, R.decide(q, shuffled, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1])
    assert np.allclose(za, R.decide(q, lower, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1])
    # the first 16 input columns of combined_projection are the hidden features (layers 1 and 3, in that order)
    q = dict(p)
    w = p["combined_projection.weight"].copy(); w[:, 16:] = 0
    q["combined_projection.weight"] = w
    zb = R.decide(q, logits, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1]
    assert np.allclose(zb, R.decide(q, logits * 0 + 1, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1])
    hs2 = hs.copy(); hs2[..., 0, :] += 3; hs2[..., 2, :] -= 2      # layers that are not selected
    assert np.allclose(zb, R.decide(q, logits, 0, hs2, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1])
    hs3 = hs.copy(); hs3[..., 1, :], hs3[..., 3, :] = hs[..., 3, :], hs[..., 1, :]
    assert not np.allclose(zb, R.decide(q, logits, 0, hs3, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1])


def test_residual_wiring_and_closed_forms():
    p, logits, hs, z = _case(False)
    # second layer of every block's MLP switched off: a block is its skip path alone
    q = dict(p)
    for i in range(3):
        q[f"backbone.blocks.{i}.mlp.3.weight"] = np.zeros_like(p[f"backbone.blocks.{i}.mlp.3.weight"])
        q[f"backbone.blocks.{i}.mlp.3.bias"] = np.zeros_like(p[f"backbone.blocks.{i}.mlp.3.bias"])
    x = R._lin(q, "combined_projection", np.concatenate([R.hidden_features(hs, (1, 3), (2, 3), 8), R._lin(q, "logits_projection", R.topk_values(logits, 5))], -1))
    x = R._lin(q, "backbone.input_projection", x)
    x = R._lin(q, "backbone.blocks.1.dim_change", R._lin(q, "backbone.blocks.0.dim_change", x))   # block 2 keeps its width: identity skip
    want = R._lin(q, "backbone.output_layer.1", R._layer_norm(q, "backbone.output_layer.0", x))[..., 0]
    assert np.allclose(R.decide(q, logits, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1], want)
    # all weights zero: the logit is the output bias, whatever comes in
    zero = {k: (np.zeros_like(v) if k.endswith(".weight") and "layer_norm" not in k and "output_layer.0" not in k else v) for k, v in p.items()}
    dec, z0 = R.decide(zero, logits, 0, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)
    ln_bias_path = R._lin(zero, "backbone.output_layer.1", np.zeros(6))   # (zero weight: bias only)
    assert np.allclose(z0, ln_bias_path[0])
    # the cap (iter_decider.py:273-274) and missing hidden states (zeros in their place, :255-256)
    dec, zc = R.decide(p, logits, 3, hs, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3, max_iter=3)
    assert not dec.any() and (zc == -10.0).all() and dec.shape == (2, 3)
    assert np.allclose(R.decide(p, logits, 0, None, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1],
                       R.decide(p, logits, 0, hs * 0, topk=5, hidden_size=8, layer_nums=(1, 3), n_blocks=3)[1])
    # a single layer passed without the layer axis counts as layer 0 of 1 (:258-259)
    one = hs[..., 1, :]
    assert np.allclose(R.hidden_features(one, (0,), (2, 3), 8), one)
