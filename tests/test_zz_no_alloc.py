"""GPU: tah_duo_decode_static (split-K partials in the library's own device buffer, no allocation) gives
bit for bit what tah_duo_decode gives with a caller workspace -- on two calls in a row, the second with a
smaller input, so that what the first call left in the shared buffer is shown not to leak into the second."""
import numpy as np
import pytest
import torch

from tests.cases import build_slabs, make_decode_case

pytestmark = pytest.mark.gpu


def _inputs(seed, lens, cap1, cap2):
    c = make_decode_case(seed, lens, 0.06, hard_new=[b % 3 == 0 for b in range(len(lens))])
    s1, s2 = build_slabs(c, cap1, cap2, device="cuda")
    nseq = len(lens)
    hr = torch.tensor(c["hard_rows"], dtype=torch.int32, device="cuda")
    slot = torch.cat([torch.arange(nseq, dtype=torch.int32, device="cuda"), hr])
    qpos1 = torch.from_numpy(c["q_pos"]).cuda()
    qpos = torch.cat([qpos1, qpos1[hr.long()]])
    qd = torch.tensor([0] * nseq + [1] * len(hr), dtype=torch.int32, device="cuda")
    q = torch.cat([c["q1"].cuda(), c["q2"].cuda()])
    return c, q, slot, qpos, qd, s1, s2


def test_decode_static_scratch_matches_workspace_entry_point():
    from tah_amd import TahDuoError, _capi, kv_cache
    g = torch.Generator().manual_seed(5)
    big = torch.randint(3000, 9000, (24,), generator=g).tolist()
    small = torch.randint(100, 2500, (5,), generator=g).tolist()
    for seed, lens, cap1, cap2 in ((71, big, 9216, 1024), (72, small, 3072, 1024)):
        print(f"static-scratch decode: seed={seed} nseq={len(lens)} cap=({cap1},{cap2})", flush=True)
        c, q, slot, qpos, qd, s1, s2 = _inputs(seed, lens, cap1, cap2)
        want, want_lse = kv_cache.decode(q, slot, qpos, s1, s2, scale=c["scale"], q_depth=qd, return_lse=True)
        out = torch.full_like(want, float("nan"))
        lse = torch.full_like(want_lse, float("nan"))
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        kv_cache.decode(q, slot, qpos, s1, s2, scale=c["scale"], q_depth=qd, out=out, lse_out=lse, static_scratch=True)
        assert torch.cuda.memory_allocated() == before  # nothing was allocated through torch either
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(lse, want_lse)
    # a request beyond the library's buffer is refused with its own error, nothing is launched
    nq = 64
    cap = 1024 * (1 + _capi.STATIC_SCRATCH_BYTES // (nq * 16 * 520))
    s1 = kv_cache.KvSlabs(1, cap, 8, with_pos=False, device="cuda")
    q = torch.zeros(nq, 16, 128, dtype=torch.bfloat16, device="cuda")
    z = torch.zeros(nq, dtype=torch.int32, device="cuda")
    with pytest.raises(TahDuoError, match="scratch"):
        kv_cache.decode(q, z, z, s1, None, scale=1.0, static_scratch=True)
