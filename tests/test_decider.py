"""tah_amd.decider.MLPIterDecider (the serving-side stand-in for tah/model/iter_decider.py:193-301) against the
float64 oracle: on the CPU execution build of the top-k kernel here, on the GPU at the released sizes."""
import pytest
import torch

from tests import decider_case as D, emu_util


# What the reference's constructor builds for its default arguments (read off iter_decider.py:205-241 and :131-175):
# the state-dict names and shapes a released iter_decider.bin holds.
REFERENCE_STATE = {
    "threshold": (),
    "logits_projection.weight": (1024, 100), "logits_projection.bias": (1024,),
    "combined_projection.weight": (256, 5120), "combined_projection.bias": (256,),
    "backbone.input_projection.weight": (256, 256), "backbone.input_projection.bias": (256,),
    "backbone.blocks.0.layer_norm.weight": (256,), "backbone.blocks.0.layer_norm.bias": (256,),
    "backbone.blocks.0.mlp.0.weight": (1024, 256), "backbone.blocks.0.mlp.0.bias": (1024,),
    "backbone.blocks.0.mlp.3.weight": (512, 1024), "backbone.blocks.0.mlp.3.bias": (512,),
    "backbone.blocks.0.dim_change.weight": (512, 256), "backbone.blocks.0.dim_change.bias": (512,),
    "backbone.blocks.1.layer_norm.weight": (512,), "backbone.blocks.1.layer_norm.bias": (512,),
    "backbone.blocks.1.mlp.0.weight": (2048, 512), "backbone.blocks.1.mlp.0.bias": (2048,),
    "backbone.blocks.1.mlp.3.weight": (256, 2048), "backbone.blocks.1.mlp.3.bias": (256,),
    "backbone.blocks.1.dim_change.weight": (256, 512), "backbone.blocks.1.dim_change.bias": (256,),
    "backbone.blocks.2.layer_norm.weight": (256,), "backbone.blocks.2.layer_norm.bias": (256,),
    "backbone.blocks.2.mlp.0.weight": (1024, 256), "backbone.blocks.2.mlp.0.bias": (1024,),
    "backbone.blocks.2.mlp.3.weight": (256, 1024), "backbone.blocks.2.mlp.3.bias": (256,),
    "backbone.output_layer.0.weight": (256,), "backbone.output_layer.0.bias": (256,),
    "backbone.output_layer.1.weight": (1, 256), "backbone.output_layer.1.bias": (1,),
}


def test_state_dict_has_the_reference_names_and_shapes():
    from tah_amd.decider import MLPIterDecider
    sd = MLPIterDecider().state_dict()
    assert {k: tuple(v.shape) for k, v in sd.items()} == REFERENCE_STATE
    assert all(v.dtype == torch.bfloat16 for v in sd.values())
    extra = MLPIterDecider(normalize_input=True).state_dict()
    assert set(extra) - set(sd) == {"layer_norm_hidden_states.weight", "layer_norm_hidden_states.bias"}
    assert tuple(extra["layer_norm_hidden_states.weight"].shape) == (4096,)


def test_cap_and_dtype_need_no_kernel():
    from tah_amd.decider import MLPIterDecider
    m = MLPIterDecider(**D.SMALL)
    logits = torch.zeros(2, 3, 50, dtype=torch.bfloat16)
    dec, z = m(logits, 3)
    assert dec.shape == (2, 3) and not dec.any() and (z == -10).all() and z.dtype == torch.bfloat16
    with pytest.raises(TypeError):
        m(logits.float(), 0)
    with pytest.raises(ValueError):
        m.hidden_features(torch.zeros(2, 3, 3, 32), (2, 3), logits)   # layer 3 of 3


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_decider_on_cpu_shim():
    with emu_util.emulated():
        for normalize in (False, True):
            m = D.make("cpu", torch.float32, seed=3, normalize_input=normalize, **D.SMALL)
            logits, hs = D.inputs("cpu", (2, 5), 300, 4, 32)
            D.check(m, logits, hs, atol=2e-4, rtol=2e-4)             # float32 layers: the top-k values are exact
            if not normalize:
                D.check(m, logits[0], None, atol=2e-4, rtol=2e-4)
                D.check(m, logits[0, 0], hs[0, 0], atol=2e-4, rtol=2e-4)  # no leading dimensions but the vocabulary's
        m = D.make("cpu", torch.bfloat16, seed=4, **D.SMALL)
        logits, hs = D.inputs("cpu", (7,), 300, 4, 32, seed=5)
        D.check(m, logits, hs, atol=0.08, rtol=0.05)                 # bf16 layers, as released


def _fused_checks(dev, cfg, V, n_layers, H, rows_list, atol, rtol):
    """Up to 32 rows of a bf16 decider: the dense layers run on tah_linear_rows (LayerNorms folded, GELU and skips in
    the launches); against the oracle like the library path, whose error on the same inputs it must not exceed by much."""
    for normalize in (False, True):
        m = D.make(dev, torch.bfloat16, seed=21, normalize_input=normalize, **cfg)
        for rows in rows_list:
            logits, hs = D.inputs(dev, (rows,), V, n_layers, H, seed=30 + rows)
            assert m.takes_fused_path(rows)
            m._plan = None
            err = D.check(m, logits, hs, atol=atol, rtol=rtol)
            assert m._plan is not None            # the chain of launches was built, i.e. taken
            m.fused_layers = False
            err_lib = D.check(m, logits, hs, atol=atol, rtol=rtol)
            m.fused_layers = True
            assert err <= 2 * err_lib + 0.02, (err, err_lib)
    # more rows than a launch takes: the library's GEMMs
    logits, hs = D.inputs(dev, (3, 15), V, n_layers, H, seed=40)
    m._plan = None
    D.check(m, logits, hs, atol=atol, rtol=rtol)
    assert m._plan is None and not m.takes_fused_path(45)
    # new weights (a state dict loaded): the packed copies follow
    logits, hs = D.inputs(dev, (9,), V, n_layers, H, seed=41)
    m = D.make(dev, torch.bfloat16, seed=22, **cfg)
    D.check(m, logits, hs, atol=atol, rtol=rtol)
    other = D.make(dev, torch.bfloat16, seed=23, **cfg)
    z_other = other(logits, 0, all_hidden_states=hs)[1]
    m.load_state_dict(other.state_dict())
    assert torch.equal(m(logits, 0, all_hidden_states=hs)[1], z_other)
    D.check(m, logits, hs, atol=atol, rtol=rtol)
    # no hidden states: zeros in their place (iter_decider.py:251-252); leading dimensions are kept
    D.check(m, logits.view(3, 3, -1), None, atol=atol, rtol=rtol)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_decider_dense_layers_on_the_linear_kernel_on_cpu_shim():
    with emu_util.emulated():
        _fused_checks("cpu", D.FUSABLE, 300, 4, 32, (7, 32, 1), atol=0.08, rtol=0.05)


@pytest.mark.gpu
def test_decider_dense_layers_on_the_linear_kernel_gpu():
    _fused_checks("cuda", D.FUSABLE, 300, 4, 32, (7, 32, 1), atol=0.08, rtol=0.05)
    _fused_checks("cuda", {}, 151936, 29, 1024, (32, 19), atol=0.06, rtol=0.03)   # the released sizes
    m = D.make("cuda", torch.bfloat16, seed=25)
    logits, hs = D.inputs("cuda", (32,), 151936, 29, 1024, seed=26)
    m(logits, 0, all_hidden_states=hs)
    with torch.cuda.device(0):
        torch.cuda.set_sync_debug_mode("error")     # the chain reads nothing back either
        try:
            m(logits, 0, all_hidden_states=hs)
        finally:
            torch.cuda.set_sync_debug_mode("default")


@pytest.mark.gpu
def test_decider_gpu_released_sizes():
    logits, hs = D.inputs("cuda", (2, 24), 151936, 29, 1024, seed=7)
    m32 = D.make("cuda", torch.float32, seed=8)
    D.check(m32, logits, hs, atol=1e-3, rtol=1e-3)
    m = D.make("cuda", torch.bfloat16, seed=9, normalize_input=True)
    D.check(m, logits, hs, atol=0.06, rtol=0.03)     # bf16 layers: measured 0.022 at most on logits up to 3
    # the same weights through a state dict, as a released decider would arrive
    from tah_amd.decider import MLPIterDecider
    again = MLPIterDecider(normalize_input=True).to("cuda")
    again.load_state_dict(m.state_dict())
    a, b = m(logits, 1, all_hidden_states=hs), again(logits, 1, all_hidden_states=hs)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    with torch.cuda.device(0):
        torch.cuda.set_sync_debug_mode("error")     # no read-back of the threshold or anything else
        try:
            m(logits, 0, all_hidden_states=hs)
        finally:
            torch.cuda.set_sync_debug_mode("default")
