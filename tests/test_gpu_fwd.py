"""GPU parity: forward kernel and pack kernels through the C ABI vs the CPU oracle."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests.cases import add_score_drift, dense_to_varlen, make_dense_case, make_varlen_case, varlen_args
from tests.gpu_util import assert_close, oracle_fwd, to_device

pytestmark = pytest.mark.gpu


def _run(dev):
    from tah_amd import ops
    out = ops.duo_fwd_varlen(*varlen_args(dev))
    torch.cuda.synchronize()
    return out


def _check(dev, out, tag):
    o1, lse1, o2, lse2 = oracle_fwd(dev)
    print(tag, "o1", assert_close(out[0], o1, tag + " o1"), "o2", assert_close(out[2], o2, tag + " o2"), flush=True)
    np.testing.assert_allclose(out[1].cpu().numpy(), lse1, atol=5e-3, rtol=1e-3)
    np.testing.assert_allclose(out[3].cpu().numpy(), lse2, atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("hq,hkv,seqlens,p,seed", [
    (16, 8, [512], 0.06, 1235),             # BASELINE config 0 shape (B=1, T=512, p=0.06)
    (16, 8, [300, 1000, 17, 129], 0.10, 2),  # ragged batch
    (8, 8, [257, 64], 0.2, 3),              # no GQA
    (16, 4, [700], 0.3, 4),                 # group of 4
    (8, 1, [130, 31], 0.5, 5),              # group of 8
    (16, 8, [1], 1.0, 6),                   # single token, hard
    (16, 8, [777], 0.0, 7),                 # no hard tokens at all
    (16, 8, [640], 1.0, 8),                 # every token hard
])
def test_fwd_matches_oracle(hq, hkv, seqlens, p, seed):
    print(f"case hq={hq} hkv={hkv} seqlens={seqlens} p={p} seed={seed}", flush=True)
    dev = to_device(make_varlen_case(seed, seqlens, p, Hq=hq, Hkv=hkv, D=128))
    _check(dev, _run(dev), "fwd")


@pytest.mark.parametrize("nats_per_key", [0.25, 0.02, 0.002])
def test_fwd_moving_softmax_reference(nats_per_key):
    """Scores that keep growing along the keys, so that the running exponent reference must follow the
    row maximum in every tile (fast drift), every few tiles, or almost never (slow drift)."""
    print(f"case drift nats_per_key={nats_per_key}", flush=True)
    dev = to_device(add_score_drift(make_varlen_case(31, [1500, 333], 0.1), nats_per_key))
    _check(dev, _run(dev), "drift")


@pytest.mark.parametrize("hq,hkv,seqlens,p,seed", [
    (32, 4, [160] * 12 + [128] * 8 + [33, 1, 97], 0.3, 41),  # 32-row tiles, many short sequences
    (16, 8, [1100, 640, 2048, 129], 0.1, 42),                # 128-row tiles
    (8, 8, [2304, 257, 4000, 4096, 4096], 0.05, 43),          # 256-row tiles
    (16, 2, [3000, 1500], 0.1, 44),                          # two kv heads
])
def test_fwd_more_tiles_than_compute_units(hq, hkv, seqlens, p, seed):
    """Batches with more query tiles than the device has compute units (several rounds of workgroups)."""
    print(f"case many-tiles hq={hq} hkv={hkv} seqlens={seqlens} p={p} seed={seed}", flush=True)
    dev = to_device(make_varlen_case(seed, seqlens, p, Hq=hq, Hkv=hkv, D=128))
    _check(dev, _run(dev), "many-tiles")


def test_fwd_cache_prefix_extra_depth1_keys():
    dev = to_device(make_varlen_case(11, [40, 1, 300], 0.3, seqlens_k=[500, 900, 300], extra_k2=100))
    _check(dev, _run(dev), "prefix")


def test_fwd_left_padded_dense_batch():
    c = make_dense_case(12, B=3, T=200, p_hard=0.15, left_pad=[0, 37, 180])
    dev = to_device(dense_to_varlen(c))
    _check(dev, _run(dev), "leftpad")


def test_fwd_strided_views_of_fused_projection():
    dev = to_device(make_varlen_case(13, [333], 0.2))
    T = dev["q1"].shape[0]
    fused = torch.zeros(T, 16 + 8 + 8, 128, dtype=torch.bfloat16, device="cuda")
    fused[:, :16], fused[:, 16:24], fused[:, 24:] = dev["q1"], dev["k1"], dev["v1"]
    dev["q1"], dev["k1"], dev["v1"] = fused[:, :16], fused[:, 16:24], fused[:, 24:]
    _check(dev, _run(dev), "strided")


def test_fwd_rejects_bad_inputs():
    from tah_amd import TahDuoError, ops
    dev = to_device(make_varlen_case(14, [10], 0.5, D=64))
    with pytest.raises(TahDuoError):
        ops.duo_fwd_varlen(*varlen_args(dev))
    cpu = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in to_device(make_varlen_case(14, [10], 0.5)).items()}
    with pytest.raises(TahDuoError):
        ops.duo_fwd_varlen(*varlen_args(cpu))


def test_fwd_full_size_prefill_vs_torch_fp32():
    """BASELINE config 1 (B=4, T=4096, p=0.06) at full size against a torch fp32 reference on the GPU."""
    dev = to_device(make_varlen_case(1235, [4096] * 4, 0.06, std=0.5))
    out = _run(dev)
    scale = dev["scale"]
    worst = [0.0, 0.0]
    for b in range(4):
        a0, a1 = int(dev["cu_q1"][b]), int(dev["cu_q1"][b + 1])
        hd = lambda x: x.float().transpose(0, 1)[None]
        k = hd(dev["k1"][a0:a1]).repeat_interleave(2, 1)
        v = hd(dev["v1"][a0:a1]).repeat_interleave(2, 1)
        ref1 = F.scaled_dot_product_attention(hd(dev["q1"][a0:a1]), k, v, is_causal=True, scale=scale)[0].transpose(0, 1)
        ma, mr = assert_close(out[0][a0:a1], ref1.cpu().numpy(), f"full o1 seq {b}")
        d0, d1 = int(dev["cu_q2"][b]), int(dev["cu_q2"][b + 1])
        pos = dev["pos_q2"][d0:d1].long()
        see = torch.cat([torch.arange(a1 - a0, device="cuda")[None] <= pos[:, None], pos[None] <= pos[:, None]], 1)
        k2 = torch.cat([k, hd(dev["k2"][d0:d1]).repeat_interleave(2, 1)], 2)
        v2 = torch.cat([v, hd(dev["v2"][d0:d1]).repeat_interleave(2, 1)], 2)
        ref2 = F.scaled_dot_product_attention(hd(dev["q2"][d0:d1]), k2, v2, attn_mask=see[None, None], scale=scale)[0].transpose(0, 1)
        ma2, mr2 = assert_close(out[2][d0:d1], ref2.cpu().numpy(), f"full o2 seq {b}")
        worst = [max(worst[0], ma, ma2), max(worst[1], mr, mr2)]
    print("full-size prefill: worst max-abs-err %.3e, worst mean-rel-err %.3e" % tuple(worst), flush=True)


@pytest.mark.parametrize("B,S,p", [(4, 4096, 0.06), (1, 8192, 0.10), (3, 50, 0.3), (2, 70000, 0.5), (1, 1, 1.0), (5, 16, 0.0)])
def test_hard_index_bit_exact(B, S, p):
    from tah_amd import ops
    g = torch.Generator().manual_seed(B * 1000 + S)
    mask = (torch.rand(B, S, generator=g) < p).cuda()
    pos, flat, seq, cu = ops.hard_index_build(mask)
    n = int(cu[-1])
    nz = mask.nonzero()
    assert torch.equal(cu.long().cpu(), torch.cat([torch.zeros(1, dtype=torch.long), torch.cumsum(mask.sum(1), 0).cpu()]))
    assert torch.equal(pos[:n].long(), nz[:, 1]) and torch.equal(seq[:n].long(), nz[:, 0])
    assert torch.equal(flat[:n].long(), nz[:, 0] * S + nz[:, 1])
    width = max(int(mask.sum(1).max()), 1)
    pad = ops.pad_rows_build(cu, seq, n, width)
    rank = torch.arange(n, device="cuda") - cu.long()[nz[:, 0]]
    assert torch.equal(pad.long(), nz[:, 0] * width + rank)


@pytest.mark.parametrize("dtype,inner", [(torch.bfloat16, (2048,)), (torch.int64, ()), (torch.uint8, (3,)), (torch.float32, (5, 2)),
                                         (torch.bfloat16, (16, 128))])
def test_rows_copy_bit_exact(dtype, inner):
    from tah_amd import ops
    g = torch.Generator().manual_seed(3)
    src = torch.randint(0, 100, (4000,) + inner, generator=g).to(dtype).cuda()
    rows = torch.randperm(4000, generator=g)[:1700].to(torch.int32).cuda()
    out = torch.zeros((1700,) + inner, dtype=dtype, device="cuda")
    ops.rows_copy(src, rows, out, None, 1700)
    assert torch.equal(out, src[rows.long()])
    back = torch.full_like(src, 7)
    ops.rows_copy(out, None, back, rows, 1700)
    want = torch.full_like(src, 7)
    want[rows.long()] = src[rows.long()]
    assert torch.equal(back, want)


def test_tolerance_against_reference_bf16_path_and_bf16_rounded_oracle():
    """What the stated mean-rel tolerance (tests/gpu_util.py) rests on, measured instead of argued, on the
    configs[1] workload (B=4, T=4096, 6 % hard, std 0.5).

    (a) The reference's own formulation in bf16 on the device -- dense additive mask, repeat_interleave GQA,
        torch SDPA in bf16 (tah_model.py:744-791 + sdpa_attention.py:79-166) -- is compared with the same fp32
        reference; the HIP kernel must be no further from fp32 than that path (5 % slack for noise).
    (b) Against the fp32 reference *rounded to bf16* (all a bf16-output kernel can return at best) the same
        comparison: the kernel is no further away than the reference's bf16 path is.  (Neither reaches 1e-3 by
        this measure: both multiply bf16 probabilities into V, which moves about 40 % of the outputs by one
        bf16 unit in the last place; measured 1.6e-3 for both.)"""
    from tests.gpu_util import errs
    dev = to_device(make_varlen_case(1235, [4096] * 4, 0.06, std=0.5))
    out = _run(dev)
    scale = dev["scale"]
    fmin = torch.finfo(torch.bfloat16).min
    tot = {"hip": [0.0, 0.0, 0], "ref_bf16": [0.0, 0.0, 0], "hip_vs_rounded": [0.0, 0.0, 0], "ref_vs_rounded": [0.0, 0.0, 0]}
    worst_abs = {"hip": 0.0, "ref_bf16": 0.0}

    def acc(name, got, want):
        d = (got.double() - want.double()).abs()
        tot[name][0] += float(d.sum()); tot[name][1] += float(want.double().abs().sum()); tot[name][2] += d.numel()
        if name in worst_abs:
            worst_abs[name] = max(worst_abs[name], float(d.max()))

    for b in range(4):
        a0, a1 = int(dev["cu_q1"][b]), int(dev["cu_q1"][b + 1])
        d0, d1 = int(dev["cu_q2"][b]), int(dev["cu_q2"][b + 1])
        hd = lambda x: x.transpose(0, 1)[None]  # [rows, H, D] -> (1, H, rows, D)
        T = a1 - a0
        ar = torch.arange(T, device="cuda")
        pos = dev["pos_q2"][d0:d1].long()
        see1 = ar[None] <= ar[:, None]
        see2 = torch.cat([ar[None] <= pos[:, None], pos[None] <= pos[:, None]], 1)
        for dt, name in ((torch.float32, "fp32"), (torch.bfloat16, "ref_bf16")):
            k = hd(dev["k1"][a0:a1]).to(dt).repeat_interleave(2, 1)
            v = hd(dev["v1"][a0:a1]).to(dt).repeat_interleave(2, 1)
            m1 = torch.zeros(see1.shape, dtype=dt, device="cuda").masked_fill(~see1, fmin if dt == torch.bfloat16 else torch.finfo(dt).min)
            r1 = F.scaled_dot_product_attention(hd(dev["q1"][a0:a1]).to(dt), k, v, attn_mask=m1[None, None], scale=scale)[0].transpose(0, 1)
            k2 = torch.cat([k, hd(dev["k2"][d0:d1]).to(dt).repeat_interleave(2, 1)], 2)
            v2 = torch.cat([v, hd(dev["v2"][d0:d1]).to(dt).repeat_interleave(2, 1)], 2)
            m2 = torch.zeros(see2.shape, dtype=dt, device="cuda").masked_fill(~see2, fmin if dt == torch.bfloat16 else torch.finfo(dt).min)
            r2 = F.scaled_dot_product_attention(hd(dev["q2"][d0:d1]).to(dt), k2, v2, attn_mask=m2[None, None], scale=scale)[0].transpose(0, 1)
            if name == "fp32":
                f1, f2 = r1, r2
            else:
                acc("ref_bf16", r1, f1); acc("ref_bf16", r2, f2)
                acc("ref_vs_rounded", r1, f1.to(torch.bfloat16)); acc("ref_vs_rounded", r2, f2.to(torch.bfloat16))
        acc("hip", out[0][a0:a1], f1); acc("hip", out[2][d0:d1], f2)
        acc("hip_vs_rounded", out[0][a0:a1], f1.to(torch.bfloat16)); acc("hip_vs_rounded", out[2][d0:d1], f2.to(torch.bfloat16))
    mr = {n: t[0] / t[1] for n, t in tot.items()}
    print("mean-rel-err vs fp32: HIP %.3e, reference bf16 path %.3e; vs bf16-rounded fp32: HIP %.3e, reference bf16 "
          "path %.3e; max-abs vs fp32: HIP %.3e, reference bf16 path %.3e" % (
              mr["hip"], mr["ref_bf16"], mr["hip_vs_rounded"], mr["ref_vs_rounded"], worst_abs["hip"], worst_abs["ref_bf16"]),
          flush=True)
    assert mr["hip"] <= 1.05 * mr["ref_bf16"], mr
    assert worst_abs["hip"] <= max(1.05 * worst_abs["ref_bf16"], 1e-2), worst_abs
    assert mr["hip_vs_rounded"] <= 1.05 * mr["ref_vs_rounded"], mr
