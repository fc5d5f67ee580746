"""tah_topk_mix (top-k softmax mix of embedding rows, tah_model.py:57-75) against its oracle: on the CPU
execution build of the kernel, and on the GPU through the C ABI."""
import numpy as np
import pytest
import torch

from oracle.topk_mix_ref import topk_mix as ref_mix
from tests import emu_util
from tests.topk_mix_cases import make_case, to_torch

GOLDEN = __import__("os").path.join(__import__("os").path.dirname(__file__), "golden", "topk_mix_small.npz")


def _check(got, want):
    got = got.float().cpu().numpy()
    tol = np.maximum(np.abs(want), 1e-3) * 2.0 ** -7  # one bf16 step: exp2-based softmax vs exp
    assert (np.abs(got - want) <= tol).all(), float(np.abs(got - want).max())
    assert (got == want).mean() > 0.97


def _run(device, seed, rows, V, H, k, **kw):
    from tah_amd import ops
    logits, emb = make_case(seed, rows, V, H, **kw)
    out = ops.topk_mix(to_torch(logits, device), to_torch(emb, device), k)
    _check(out, ref_mix(logits, emb, k))


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
@pytest.mark.parametrize("seed,rows,V,H,k,kw", [
    (0, 2, 700, 64, 100, {}), (1, 1, 9000, 32, 17, dict(ties=0.05)), (2, 2, 90, 16, 100, {}), (3, 1, 17000, 256, 100, {}),
    (4, 1, 1003, 8, 200, dict(ties=0.3)),
    (5, 1, 17000, 16, 50, dict(ties=0.2)),   # 3400 equal logits at the threshold: more than the candidate list holds
])
def test_topk_mix_on_cpu_shim(seed, rows, V, H, k, kw):
    with emu_util.emulated():
        _run("cpu", seed, rows, V, H, k, **kw)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_topk_mix_golden_and_row_enable_on_cpu_shim():
    from tah_amd import ops
    z = np.load(GOLDEN)
    with emu_util.emulated():
        out = ops.topk_mix(to_torch(z["logits"], "cpu"), to_torch(z["emb"], "cpu"), int(z["k"]))
        assert np.array_equal(out.float().numpy(), z["out"])
        en = torch.tensor([1, 0, 1], dtype=torch.uint8)
        keep = torch.full((3, z["emb"].shape[1]), 7.0, dtype=torch.bfloat16)
        ops.topk_mix(to_torch(z["logits"], "cpu"), to_torch(z["emb"], "cpu"), int(z["k"]), row_enable=en, out=keep)
        # rows that are not enabled written as zeros, and the rows once more in the linear-layer kernels' operand order
        H = z["emb"].shape[1]
        zeroed = torch.full((3, H), 7.0, dtype=torch.bfloat16)
        packed = torch.full((32 * H,), 5.0, dtype=torch.bfloat16) if H % 32 == 0 else None
        ops.topk_mix(to_torch(z["logits"], "cpu"), to_torch(z["emb"], "cpu"), int(z["k"]), row_enable=en, out=zeroed, out_packed=packed,
                     zero_disabled=True)
    assert np.array_equal(keep[0].float().numpy(), z["out"][0]) and (keep[1] == 7).all()
    assert torch.equal(zeroed[0], keep[0]) and torch.equal(zeroed[2], keep[2]) and not zeroed[1].any()
    if packed is not None:
        from tests.test_linear_rows import unpack_rows
        rows = unpack_rows(packed, H)
        assert torch.equal(rows[:3], zeroed) and (rows[3:] == 5).all()


def test_oracle_reproduces_golden():
    z = np.load(GOLDEN)
    assert np.array_equal(ref_mix(z["logits"], z["emb"], int(z["k"])), z["out"])


@pytest.mark.gpu
@pytest.mark.parametrize("seed,rows,V,H,k,kw", [
    (10, 32, 151936, 2048, 100, {}),                 # the end-to-end workload's shape
    (11, 5, 151936, 2048, 100, dict(ties=0.02)),     # thousands of equal logits around the 100th place
    (12, 3, 50000, 256, 1, {}), (13, 4, 777, 64, 100, dict(ties=0.2)), (14, 2, 64, 128, 100, {}), (15, 7, 20001, 1024, 256, {}),
])
def test_topk_mix_gpu(seed, rows, V, H, k, kw):
    print(f"topk_mix case seed={seed} rows={rows} V={V} H={H} k={k} {kw}", flush=True)
    _run("cuda", seed, rows, V, H, k, **kw)


@pytest.mark.gpu
def test_topk_mix_gpu_vs_torch_ops_on_device_and_strided_logits():
    """Against the reference's call sequence in torch on the device (distinct values: no tie to break), with the
    logits a strided slice of a larger buffer."""
    from tah_amd import ops
    logits, emb = make_case(20, 6, 4001, 512, distinct=True)
    buf = torch.zeros(6, 4100, dtype=torch.bfloat16, device="cuda")
    buf[:, 3:4004] = to_torch(logits, "cuda")
    lg, em = buf[:, 3:4004], to_torch(emb, "cuda")
    out = ops.topk_mix(lg, em, 100)
    tv, ti = torch.topk(lg, k=100, dim=-1)
    want = torch.sum(torch.softmax(tv, -1).unsqueeze(-1) * em[ti], dim=-2).to(em.dtype)
    _check(out, want.float().cpu().numpy())
    z = np.load(GOLDEN)
    out = ops.topk_mix(to_torch(z["logits"], "cuda"), to_torch(z["emb"], "cuda"), int(z["k"]))
    assert np.array_equal(out.float().cpu().numpy(), z["out"])


def _values_check(device, V=3000, rows=3, k=100):
    """The top-k logits themselves, largest first, equal torch.topk's values to the bit (ties make the indices a
    matter of choice, the values not): alone and next to the mix; more places than vocabulary entries."""
    from tah_amd import ops
    g = torch.Generator().manual_seed(V + rows)
    logits = (torch.randn(rows, V, generator=g) * 3).to(torch.bfloat16)
    logits[0, ::7] = logits[0, 0]                      # a plateau
    logits[-1] = torch.randint(-2, 3, (V,), generator=g).to(torch.bfloat16)   # five distinct values: ties everywhere
    emb = torch.randn(V, 64, generator=g).to(torch.bfloat16)
    want = torch.topk(logits.float(), min(k, V), dim=-1).values.to(torch.bfloat16)
    ld, ed = logits.to(device), emb.to(device)
    got = ops.topk_values(ld, k)
    assert got.shape == want.shape and torch.equal(got.cpu(), want)
    vals = torch.zeros(rows, min(k, V), dtype=torch.bfloat16, device=device)
    mix = ops.topk_mix(ld, ed, k, values_out=vals)
    assert torch.equal(vals.cpu(), want) and torch.equal(mix, ops.topk_mix(ld, ed, k))
    v2, i2 = ops.topk(ld, k)                                # with the indices: the values sit there, equal ones by ascending index
    assert torch.equal(v2.cpu(), want) and torch.equal(torch.gather(logits, 1, i2.cpu().long()), want)
    for r in range(rows):
        vv, ii = want[r].float(), i2[r].cpu()
        assert all(vv[j] > vv[j + 1] or ii[j] < ii[j + 1] for j in range(len(ii) - 1))
        kth = vv[-1]
        taken = set(ii[vv == kth].tolist())
        ties = (logits[r].float() == kth).nonzero().flatten().tolist()
        assert taken == set(ties[:len(taken)])               # at the k-th place the lower indices
    small = ops.topk_values(ld[:, :40].contiguous(), 100)   # more places than entries: every entry, sorted
    assert torch.equal(small.cpu(), torch.sort(logits[:, :40].float(), dim=-1, descending=True).values.to(torch.bfloat16))


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_topk_values_on_cpu_shim():
    with emu_util.emulated():
        _values_check("cpu", rows=2)
        _values_check("cpu", V=9000, rows=1, k=17)


@pytest.mark.gpu
def test_topk_values_gpu():
    _values_check("cuda")
    _values_check("cuda", V=151936, rows=40, k=100)
    _values_check("cuda", V=151936, rows=2, k=256)


def _silu_mul_check(device):
    """tah_silu_mul against torch's own silu and product in bf16 (the eager modules' arithmetic; a library routine)."""
    import torch.nn.functional as F

    from tah_amd import ops
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn(5, 2 * 1536, generator=g) * 2).to(torch.bfloat16).to(device)
    got = ops.silu_mul(gu)
    want = F.silu(gu[:, :1536]) * gu[:, 1536:]
    d = (got.float() - want.float()).abs()
    assert (d <= want.float().abs() * 2.0 ** -7 + 1e-30).all()  # exp2-based sigmoid: at most one bf16 step
    assert (got == want).float().mean() > 0.98


def _silu_mul_normed_check(device):
    """The MLP's input norm folded in: equals scaling gate and up by the row's rsqrt(mean(x^2) + eps) first."""
    from tah_amd import ops
    g = torch.Generator().manual_seed(4)
    gu = (torch.randn(5, 2 * 1536, generator=g) * 9).to(torch.bfloat16)
    x = (torch.randn(5, 640, generator=g) * 5).to(torch.bfloat16)
    r = torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6)
    scaled = (gu.double() * r).to(torch.bfloat16)
    got = ops.silu_mul(gu.to(device), norm_input=x.to(device), norm_eps=1e-6).cpu()
    want = ops.silu_mul(scaled.to(device)).cpu()
    assert (got == want).float().mean() > 0.98   # one bf16 step where the last bit of r differs
    assert torch.allclose(got.float(), want.float(), rtol=2.0 ** -6, atol=1e-30)


def _packed_rows_check(device):
    """The rows once more in the operand order of the linear-layer kernels, rows that are not enabled as zeros."""
    from tah_amd import ops
    from tests.test_linear_rows import unpack_rows
    g = torch.Generator().manual_seed(8)
    logits = torch.randn(5, 300, generator=g).to(torch.bfloat16).to(device)
    emb = torch.randn(300, 64, generator=g).to(torch.bfloat16).to(device)
    en = torch.tensor([1, 1, 0, 1, 0], dtype=torch.bool, device=device)
    want = ops.topk_mix(logits, emb, 20, row_enable=en)
    out = torch.full((5, 64), 3.0, dtype=torch.bfloat16, device=device)
    packed = torch.full((32 * 64,), 3.0, dtype=torch.bfloat16, device=device)
    ops.topk_mix(logits, emb, 20, row_enable=en, out=out, out_packed=packed, zero_disabled=True)
    rows = unpack_rows(packed.cpu(), 64)
    assert torch.equal(out, want) and not out[2].any() and torch.equal(rows[:5], out.cpu()) and (rows[5:] == 3).all()


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_silu_mul_on_cpu_shim():
    with emu_util.emulated():
        _silu_mul_check("cpu")
        _silu_mul_normed_check("cpu")
        _packed_rows_check("cpu")


@pytest.mark.gpu
def test_silu_mul_gpu():
    _silu_mul_check("cuda")
    _silu_mul_normed_check("cuda")
    _packed_rows_check("cuda")
