"""Decode and KV-append kernels on the CPU execution shim against the oracle.  No GPU."""
import numpy as np
import pytest
import torch

from oracle import duo_oracle as O
from tests import emu_util
from tests.cases import build_slabs, make_decode_case

pytestmark = pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")


def oracle_decode(c):
    f = lambda x: x.float().numpy()
    nseq = len(c["lens"])
    o0, l0 = O.duo_decode_f64(f(c["q1"]), f(c["k1"]), f(c["v1"]), c["cu_k1"], f(c["k2"]), f(c["v2"]), c["pos_k2"],
                              c["cu_k2"], c["q_pos"], [0] * nseq, c["scale"])
    hr = c["hard_rows"]
    q2full = np.zeros((nseq,) + tuple(c["q2"].shape[1:]))
    q2full[hr] = f(c["q2"])
    o1, l1 = O.duo_decode_f64(q2full, f(c["k1"]), f(c["v1"]), c["cu_k1"], f(c["k2"]), f(c["v2"]), c["pos_k2"],
                              c["cu_k2"], c["q_pos"], [1] * nseq, c["scale"])
    return o0, l0, o1[hr], l1[hr]


# The last case has 16 (query, kv head) pairs: in the CPU execution build such calls run one workgroup per pair over
# both segments (duo_decode_whole_kernel; the MI355X build does from 256 pairs on, see the GPU tests).
@pytest.mark.parametrize("hq,hkv,lens", [(2, 1, [700, 3, 513]), (4, 1, [40]), (2, 2, [1030]), (8, 1, [70, 5]),
                                         (16, 8, [150, 37])])
def test_decode_and_append_on_cpu_shim(hq, hkv, lens):
    from tah_amd import kv_cache
    c = make_decode_case(20 + hq, lens, 0.2, Hq=hq, Hkv=hkv, hard_new=[True] + [False] * (len(lens) - 1))
    with emu_util.emulated():
        s1, s2 = build_slabs(c, 1100, 600)
        assert s1.len.tolist() == lens and s2.len.tolist() == np.diff(c["cu_k2"]).tolist()
        assert int(s1.overflow) == 0
        nseq = len(lens)
        slot = torch.arange(nseq, dtype=torch.int32)
        qpos = torch.from_numpy(c["q_pos"])
        o0, l0 = kv_cache.decode(c["q1"], slot, qpos, s1, None, scale=c["scale"], depth=0, return_lse=True)
        hr = torch.tensor(c["hard_rows"], dtype=torch.int32)
        o1, l1 = kv_cache.decode(c["q2"], hr, qpos[hr.long()], s1, s2, scale=c["scale"], depth=1, return_lse=True)
        # both depths in one launch
        qd = torch.tensor([0] * nseq + [1] * len(hr), dtype=torch.int32)
        packed = torch.full((32 * hq * 128,), 3.0, dtype=torch.bfloat16) if nseq + len(hr) <= 32 else None
        om = kv_cache.decode(torch.cat([c["q1"], c["q2"]]), torch.cat([slot, hr]), torch.cat([qpos, qpos[hr.long()]]),
                             s1, s2, scale=c["scale"], q_depth=qd, out_packed=packed)
        # a query without a sequence (slot -1, as a generation loop marks its finished rows): zeros, -inf, nothing read
        gone = slot.clone()
        gone[0] = -1
        og, lg = kv_cache.decode(c["q1"], gone, qpos, s1, None, scale=c["scale"], depth=0, return_lse=True)
        assert not og[0].any() and torch.isinf(lg[0]).all() and torch.equal(og[1:], o0[1:]) and torch.equal(lg[1:], l0[1:])
    # the same output as the rows operand of the o projection; rows past the last query are left alone
    if packed is not None:
        from tests.test_linear_rows import unpack_rows
        rows = unpack_rows(packed, hq * 128)
        assert torch.equal(rows[:om.shape[0]], om.reshape(om.shape[0], -1)) and (rows[om.shape[0]:] == 3.0).all()
    w0, wl0, w1, wl1 = oracle_decode(c)
    np.testing.assert_allclose(o0.float().numpy(), w0, atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(l0.numpy(), wl0, atol=2e-3, rtol=1e-3)
    np.testing.assert_allclose(o1.float().numpy(), w1, atol=2e-2, rtol=2e-2)
    np.testing.assert_allclose(l1.numpy(), wl1, atol=2e-3, rtol=1e-3)
    assert torch.equal(om[:nseq], o0)
    if nseq * hkv < 16:
        assert torch.equal(om[nseq:], o1)
    else:  # the depth-1 query alone went through split-K, in the joint call through the one-workgroup kernel: other sum order
        np.testing.assert_allclose(om[nseq:].float().numpy(), o1.float().numpy(), atol=2e-2, rtol=2e-2)


def test_append_is_exact_and_flags_overflow():
    from tah_amd.kv_cache import KvSlabs
    with emu_util.emulated():
        s = KvSlabs(3, 5, 2, with_pos=True, device="cpu")
        g = torch.Generator().manual_seed(0)
        k = torch.randn(6, 2, 128, generator=g).to(torch.bfloat16)
        v = torch.randn(6, 2, 128, generator=g).to(torch.bfloat16)
        pos = torch.arange(6, dtype=torch.int32) * 3
        # rows 0-1 -> slot 2, rows 2-5 -> slot 0
        s.append(k, v, torch.tensor([0, 2, 6], dtype=torch.int32), pos_new=pos, slot_of=torch.tensor([2, 0], dtype=torch.int32))
        assert s.len.tolist() == [4, 0, 2]
        assert torch.equal(s.k[2, :, :2], k[:2].transpose(0, 1)) and torch.equal(s.v[0, :, :4], v[2:].transpose(0, 1))
        assert s.pos[2, :2].tolist() == [0, 3] and s.pos[0, :4].tolist() == [6, 9, 12, 15]
        assert int(s.overflow) == 0
        s.append(k[:3], v[:3], torch.tensor([0, 3], dtype=torch.int32), pos_new=pos[:3], slot_of=torch.tensor([0], dtype=torch.int32))
        assert s.len.tolist() == [5, 0, 2] and int(s.overflow) == 1
        assert torch.equal(s.k[0, :, 4], k[0])


def test_fused_decode_step_equals_prep_then_decode_on_cpu_shim():
    """16 (query, kv head) pairs: the CPU execution build takes such calls in one launch."""
    from tests import decode_step_case
    from tah_amd import kv_cache
    with emu_util.emulated():
        assert kv_cache.decode_step_supported(2, 16, 8, 128) and not kv_cache.decode_step_supported(1, 16, 8, 128)
        assert not kv_cache.decode_step_supported(2, 32, 8, 128)  # four query heads per kv head
        decode_step_case.run("cpu", B=3, hq=16, hkv=8, seed=5)
        decode_step_case.run("cpu", B=2, hq=8, hkv=8, seed=6, full_slab=True)
        decode_step_case.run_mixed("cpu", B=4, hq=8, hkv=8, seed=7)
