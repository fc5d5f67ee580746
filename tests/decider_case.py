"""Shared by the CPU and GPU tests of the iteration decider: a decider with random weights, inputs, and what the
oracle (oracle/decider_ref.py, float64) says about them."""
import numpy as np
import torch

from oracle import decider_ref as R

SMALL = dict(topk=10, hidden_states_size=32, hidden_states_layer_nums=(1, 3), hidden_dims=(16, 32, 16), expansion_factor=2)
# every width a multiple of 32: up to 32 rows of a bf16 copy go through the linear-layer kernel, not the library
FUSABLE = dict(topk=10, hidden_states_size=32, hidden_states_layer_nums=(1, 3), hidden_dims=(32, 64, 32), expansion_factor=2)


def make(device, dtype, seed=0, normalize_input=False, threshold=0.5, **cfg):
    from tah_amd.decider import MLPIterDecider
    torch.manual_seed(seed)
    m = MLPIterDecider(normalize_input=normalize_input, threshold=threshold, dtype=dtype, **cfg)
    with torch.no_grad():  # biases and norms away from their trivial initial values
        for n, prm in m.named_parameters():
            if n.endswith(".bias") or "layer_norm" in n or "output_layer.0" in n:
                prm.add_(torch.randn_like(prm) * 0.3)
    return m.to(device).eval()


def state64(m):
    return {k: v.detach().float().cpu().numpy().astype(np.float64) for k, v in m.state_dict().items()}


def inputs(device, lead, V, n_layers, H, seed=1):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn(*lead, V, generator=g) * 4).to(torch.bfloat16)
    hs = torch.randn(*lead, n_layers, H, generator=g).to(torch.bfloat16)
    return logits.to(device), hs.to(device)


def oracle(m, logits, hs, iter_depth=0):
    n_blocks = len(m.backbone["blocks"])
    return R.decide(state64(m), logits.float().cpu().numpy(), iter_depth, None if hs is None else hs.float().cpu().numpy(),
                    topk=m.topk, hidden_size=m.hidden_states_size, layer_nums=m.hidden_states_layer_nums, n_blocks=n_blocks,
                    normalize_input=m.normalize_input, max_iter=m.max_iter)


def check(m, logits, hs, *, atol, rtol):
    """Decision logits against the oracle; decisions equal wherever the oracle's probability is not within the
    tolerance of the threshold."""
    dec, z = m(logits, 0, all_hidden_states=hs)
    want_dec, want_z = oracle(m, logits, hs)
    z = z.float().cpu().numpy()
    assert z.shape == want_z.shape and dec.shape == want_dec.shape and dec.dtype == torch.bool
    err = np.abs(z - want_z)
    assert (err <= atol + rtol * np.abs(want_z)).all(), float(err.max())
    clear = np.abs(want_z - np.log(float(m.threshold) / (1 - float(m.threshold)))) > 2 * (atol + rtol * np.abs(want_z))
    assert clear.any() and (dec.cpu().numpy()[clear] == want_dec[clear]).all()
    return float(err.max())
