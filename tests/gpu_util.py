"""Helpers for the GPU parity tests: move cases to the device, call the oracle, error metrics."""
from __future__ import annotations

import numpy as np
import torch

from oracle import duo_ref
from tests.cases import varlen_args

# Stated tolerance of the bf16 path against an fp32/float64 reference evaluated on the same
# bf16-rounded inputs.  max-abs-err <= 2e-2.  mean-rel-err = mean|a-b| / mean|b| <= 3e-3:
# rounding the exact result to bf16 (8 significant bits) already costs 2^-9/1.44 = 1.4e-3 by
# this measure, and rounding the probabilities to bf16 for the PV MFMA adds about as much
# again, so ~2e-3 is what any bf16-in/bf16-out flash kernel measures.
MAX_ABS_TOL = 2e-2
MEAN_REL_TOL = 3e-3


def to_device(case, device="cuda"):
    out = {}
    for k, v in case.items():
        if isinstance(v, np.ndarray):
            out[k] = torch.from_numpy(v.copy()).to(device)
        elif torch.is_tensor(v):
            out[k] = v.to(torch.bfloat16).to(device)
        else:
            out[k] = v
    return out


def host_args(dev):
    return [a.float().cpu().numpy() if torch.is_tensor(a) and a.is_floating_point() else
            (a.cpu().numpy() if torch.is_tensor(a) else a) for a in varlen_args(dev)]


def oracle_fwd(dev):
    return duo_ref.fwd(*host_args(dev))


def errs(got: torch.Tensor, want) -> tuple:
    g = got.float().cpu().numpy().astype(np.float64)
    w = np.asarray(want, dtype=np.float64)
    if w.size == 0:
        return 0.0, 0.0
    d = np.abs(g - w)
    return float(d.max()), float(d.mean() / max(np.abs(w).mean(), 1e-30))


def assert_close(got, want, what, max_abs=MAX_ABS_TOL, mean_rel=MEAN_REL_TOL):
    ma, mr = errs(got, want)
    assert ma <= max_abs and mr <= mean_rel, f"{what}: max-abs-err {ma:.3e} (tol {max_abs}), mean-rel-err {mr:.3e} (tol {mean_rel})"
    return ma, mr
