"""GPU parity: decode split-K kernel and KV append through the C ABI vs the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import duo_ref as R
from tests.cases import build_slabs, make_decode_case
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu


def oracle_decode_c(c):
    """Decode rows via the C oracle: one depth-0 query row per sequence (bottom-right aligned against the
    whole depth-0 segment) and one depth-1 row per hard sequence at the last position."""
    f = lambda x: x.float().numpy()
    nseq = len(c["lens"])
    hr = c["hard_rows"]
    cu_q1 = np.arange(nseq + 1, dtype=np.int32)
    cu_q2 = np.concatenate([[0], np.cumsum([1 if b in hr else 0 for b in range(nseq)])]).astype(np.int32)
    pos_q2 = c["q_pos"][hr]
    o1, lse1, o2, lse2 = R.fwd(f(c["q1"]), f(c["k1"]), f(c["v1"]), cu_q1, c["cu_k1"], f(c["q2"]), f(c["k2"]), f(c["v2"]),
                               pos_q2, c["pos_k2"], cu_q2, c["cu_k2"], c["scale"])
    return o1, lse1.T, o2, lse2.T


def run_decode(c, cap1, cap2, fused):
    from tah_amd import kv_cache
    s1, s2 = build_slabs(c, cap1, cap2, device="cuda")
    nseq = len(c["lens"])
    slot = torch.arange(nseq, dtype=torch.int32, device="cuda")
    qpos = torch.from_numpy(c["q_pos"]).cuda()
    hr = torch.tensor(c["hard_rows"], dtype=torch.int32, device="cuda")
    q1, q2 = c["q1"].cuda(), c["q2"].cuda()
    if fused:
        qd = torch.tensor([0] * nseq + [1] * len(hr), dtype=torch.int32, device="cuda")
        nq = nseq + len(hr)  # up to 32 queries the output is also written as the o projection's rows operand
        packed = torch.zeros(32 * q1.shape[1] * q1.shape[2], dtype=torch.bfloat16, device="cuda") if nq <= 32 else None
        o, lse = kv_cache.decode(torch.cat([q1, q2]), torch.cat([slot, hr]), torch.cat([qpos, qpos[hr.long()]]), s1, s2,
                                 scale=c["scale"], q_depth=qd, return_lse=True, out_packed=packed)
        if packed is not None:
            from tests.test_linear_rows import unpack_rows
            rows = unpack_rows(packed.cpu(), q1.shape[1] * q1.shape[2])
            assert torch.equal(rows[:nq], o.cpu().reshape(nq, -1)) and not rows[nq:].any()
        out = o[:nseq], lse[:nseq], o[nseq:], lse[nseq:]
    else:
        o0, l0 = kv_cache.decode(q1, slot, qpos, s1, None, scale=c["scale"], depth=0, return_lse=True)
        if len(hr):
            o1, l1 = kv_cache.decode(q2, hr, qpos[hr.long()], s1, s2, scale=c["scale"], depth=1, return_lse=True)
        else:
            o1, l1 = q2, torch.zeros(0, q2.shape[1], device="cuda")
        out = o0, l0, o1, l1
    torch.cuda.synchronize()
    assert int(s1.overflow) == 0 and int(s2.overflow) == 0
    assert s1.len.cpu().tolist() == list(c["lens"])
    return out


@pytest.mark.parametrize("hq,hkv,lens,fused", [
    (16, 8, [700, 3, 513, 512, 1], False),
    (16, 8, [1030, 2049], True),
    (8, 8, [300], False),
    (16, 4, [777, 64], True),
    (16, 2, [1500, 33], True),   # group of 8 query heads per kv head
    # 256 or more (query, kv head) pairs and slabs of at most 4096 rows: one workgroup per pair, no merge launch
    (16, 8, [1 + (211 * i) % 2000 for i in range(32)], True),
    (16, 8, [1 + (97 * i) % 1200 for i in range(40)], False),
    (8, 8, [5 + (53 * i) % 700 for i in range(32)], True),
    (32, 4, [1 + (151 * i) % 900 for i in range(64)], False),  # group of 8
])
def test_decode_matches_oracle(hq, hkv, lens, fused):
    print(f"decode case hq={hq} hkv={hkv} lens={lens} fused={fused}", flush=True)
    c = make_decode_case(30 + hq + len(lens), lens, 0.2, Hq=hq, Hkv=hkv, hard_new=[b % 2 == 0 for b in range(len(lens))])
    got = run_decode(c, 2100, 700, fused)
    w0, wl0, w1, wl1 = oracle_decode_c(c)
    print("o depth0", assert_close(got[0], w0, "decode o depth0"), "o depth1", assert_close(got[2], w1, "decode o depth1"))
    np.testing.assert_allclose(got[1].cpu().numpy(), wl0, atol=5e-3, rtol=1e-3)
    np.testing.assert_allclose(got[3].cpu().numpy(), wl1, atol=5e-3, rtol=1e-3)


def test_decode_full_size_config():
    """BASELINE config 2: 64 sequences, context uniform in [1024, 16384], 6 % depth-1 rows, bf16."""
    g = torch.Generator().manual_seed(1236)
    lens = torch.randint(1024, 16385, (64,), generator=g).tolist()
    c = make_decode_case(1236, lens, 0.06)
    print("full-size decode: sum(L) =", sum(lens), "hard rows:", c["hard_rows"], flush=True)
    got = run_decode(c, 16384, 2048, True)
    w0, wl0, w1, wl1 = oracle_decode_c(c)
    print("o depth0", assert_close(got[0], w0, "decode o depth0"), "o depth1", assert_close(got[2], w1, "decode o depth1"))
    np.testing.assert_allclose(got[1].cpu().numpy(), wl0, atol=5e-3, rtol=1e-3)
    np.testing.assert_allclose(got[3].cpu().numpy(), wl1, atol=5e-3, rtol=1e-3)


def test_decode_query_before_end_of_cache_sees_prefix_only():
    """A query at position p < len-1 sees rows 0..p only (depth 0) and depth-1 rows with pos <= p."""
    from tah_amd import kv_cache
    c = make_decode_case(41, [900], 0.3, hard_new=[True])
    s1, s2 = build_slabs(c, 1024, 512, device="cuda")
    p = 555
    n2 = int((c["pos_k2"] <= p).sum())
    short = dict(c, lens=[p + 1], k1=c["k1"][: p + 1], v1=c["v1"][: p + 1], cu_k1=np.array([0, p + 1], np.int32),
                 k2=c["k2"][:n2], v2=c["v2"][:n2], pos_k2=c["pos_k2"][:n2], cu_k2=np.array([0, n2], np.int32),
                 q_pos=np.array([p], np.int32))
    w0, _, w1, _ = oracle_decode_c(short)
    z = torch.zeros(1, dtype=torch.int32, device="cuda")
    o0 = kv_cache.decode(c["q1"].cuda(), z, z + p, s1, None, scale=c["scale"], depth=0)
    o1 = kv_cache.decode(c["q2"].cuda(), z, z + p, s1, s2, scale=c["scale"], depth=1)
    assert_close(o0, w0, "prefix depth0")
    assert_close(o1, w1, "prefix depth1")


def test_decode_rejects_small_workspace_and_bad_shapes():
    import ctypes
    from tah_amd import _capi, _lib
    lib = _capi.bind(ctypes.CDLL(_lib.LIB_PATH))
    a = _capi.DuoDecodeArgs()
    a.d, a.nq, a.hq, a.hkv = 64, 1, 2, 1
    assert lib.tah_duo_decode(ctypes.byref(a), None) == -2
    a.d = 128
    assert lib.tah_duo_decode(ctypes.byref(a), None) == -1
    assert lib.tah_duo_decode_workspace_bytes(64, 16, 16384, 2048) == 64 * 16 * (16 + 2) * 130 * 4


@pytest.mark.parametrize("B,hq,hkv", [(32, 16, 8), (40, 8, 8), (64, 8, 4)])
def test_fused_decode_step_equals_prep_then_decode(B, hq, hkv):
    """tah_duo_decode_step against tah_qk_prep + tah_duo_decode: bit for bit (outputs, cache rows, positions, lengths)."""
    from tests import decode_step_case
    from tah_amd import kv_cache
    print(f"fused decode step B={B} hq={hq} hkv={hkv}", flush=True)
    assert kv_cache.decode_step_supported(B, hq, hkv, 4096) and not kv_cache.decode_step_supported(B, hq, hkv, 4097)
    assert not kv_cache.decode_step_supported(B, 4 * hkv, hkv, 4096)  # four query heads per kv head: the two calls
    decode_step_case.run("cuda", B=B, hq=hq, hkv=hkv, seed=B + hq, max_len=3000, hidden=2048, cap1=4096, cap2=1024)
    decode_step_case.run("cuda", B=B, hq=hq, hkv=hkv, seed=B + hq + 1, max_len=500, hidden=512, cap2=512, full_slab=True)
    decode_step_case.run_mixed("cuda", B=B, hq=hq, hkv=hkv, seed=B + hq + 2, max_len=3000, hidden=2048, cap1=4096, cap2=1024)
