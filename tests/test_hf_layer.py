"""The fused attention-layer forward against the transformers module's own forward."""
import pytest
import torch

from tests import emu_util
from tests.hf_layer_case import run, run_prefill_then_decode


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
