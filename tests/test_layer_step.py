"""Decode loop of one attention layer (q/k preparation + append, then decode) against a plain restatement."""
import pytest

from tests import emu_util
from tests.layer_step_case import run


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_layer_decode_loop_on_cpu_shim():
    from tah_amd.kv_cache import KvSlabs, decode, qk_norm_rope
    with emu_util.emulated():
        worst = run("cpu", qk_norm_rope, KvSlabs, decode, B=2, hq=2, hkv=1, prompt=(9, 3), steps=2, cap=16)
    assert worst <= 2e-2, worst


@pytest.mark.gpu
def test_layer_decode_loop_gpu():
    from tah_amd.kv_cache import KvSlabs, decode, qk_norm_rope
    worst = run("cuda", qk_norm_rope, KvSlabs, decode, B=5, hq=16, hkv=8, prompt=(700, 5, 64, 1, 1300), steps=4, cap=1400, seed=3)
    print("layer decode loop: worst abs error", worst, flush=True)
    assert worst <= 2e-2, worst
