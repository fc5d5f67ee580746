"""The fused attention-layer forward against the transformers module's own forward."""
import pytest
import torch

from tests import emu_util
from tests.hf_layer_case import run, run_prefill_then_decode, run_training_step


def _check(got, want):
    err = (got - want).abs().max().item()
    ref = want.abs().max().item()
    assert err <= 2e-2 * max(ref, 1.0), (err, ref)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_fused_layer_forward_on_cpu_shim():
    with emu_util.emulated():
        got, want = run("cpu", B=2, T=21)
    _check(got, want)


@pytest.mark.gpu
def test_fused_layer_forward_gpu():
    got, want = run("cuda", B=3, T=300)
    _check(got, want)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_fused_layer_prefill_then_decode_on_cpu_shim():
    with emu_util.emulated():
        outs = run_prefill_then_decode("cpu", B=2, T=9, steps=2)
    for ref, got in outs:
        _check(got, ref)


@pytest.mark.gpu
def test_fused_layer_prefill_then_decode_gpu():
    for ref, got in run_prefill_then_decode("cuda", B=3, T=200, steps=3):
        _check(got, ref)


def _check_training(outs):
    """Both runs are bf16 end to end (the module's own backward through eager bf16 modules): gradients agree to 4 % of
    their largest entry, the norm weights' (sums over every token and head) to 6 %."""
    (y0, dx0, g0), (y1, dx1, g1) = outs
    _check(y1, y0)
    assert (dx1 - dx0).abs().max() <= 4e-2 * dx0.abs().max()
    assert set(g0) == set(g1) and {"q_norm.weight", "k_norm.weight", "q_proj.weight", "o_proj.weight"} <= set(g0)
    for n in g0:
        tol = 6e-2 if "norm" in n else 4e-2
        assert (g1[n] - g0[n]).abs().max() <= tol * g0[n].abs().max(), (n, float((g1[n] - g0[n]).abs().max() / g0[n].abs().max()))


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_fused_layer_training_step_on_cpu_shim():
    with emu_util.emulated():
        _check_training(run_training_step("cpu", B=2, T=21))


@pytest.mark.gpu
def test_fused_layer_training_step_gpu():
    _check_training(run_training_step("cuda", B=3, T=300))


def _check_model(outs):
    (ref0, ref1), (got0, got1) = outs
    for got, want in ((got0, ref0), (got1, ref1)):
        err = (got - want).abs().max().item()
        ref = want.abs().max().item()
        assert err <= 3e-2 * max(ref, 1.0), (err, ref)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_patched_model_two_depths_on_cpu_shim():
    from tests.hf_model_case import run as run_model

    with emu_util.emulated():
        outs = run_model("cpu", B=2, T=12, layers=2)
    _check_model(outs)


@pytest.mark.gpu
def test_patched_model_two_depths_gpu():
    from tests.hf_model_case import run as run_model

    _check_model(run_model("cuda", B=3, T=150, layers=2))
