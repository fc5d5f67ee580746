"""Prefill then single-token decode steps at both depths through ``TaHDuoCache`` (slabs on) and
``duo_attention_forward``, next to the reference formulation (dense mask + concatenating cache + SDPA,
oracle.duo_oracle) on the same inputs.  The flow is the generate loop's (tah/model/utils.py:235-256 calling
tah_model.py:580-623): depth 0 for every row, then ``gather_active`` packs the hard rows to (B, 1) with the
other rows as pad rows (tah_model.py:116-118) and the depth-1 write appends for all B rows
(causal_cache.py:84-97).  Shared by the CPU-shim test and the GPU test."""
import types

import numpy as np
import torch

from oracle import duo_oracle as O
from tests.cases import make_dense_case


def _layer(layer_idx=0):
    return types.SimpleNamespace(layer_idx=layer_idx, num_key_value_groups=2)


def run(device, *, T0=20, steps=3, B=2, left_pad=(0, 5), seed=34, Hq=2, Hkv=1, force_hard=None, p_hard=0.3):
    """Returns the cache; asserts outputs against the oracle after every step."""
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.cache import TaHDuoCache
    from tah_amd.pack import gather_active

    c = make_dense_case(seed, B=B, T=T0 + steps, p_hard=p_hard, Hq=Hq, Hkv=Hkv, D=128, left_pad=list(left_pad))
    if force_hard is not None:  # per decode step: which batch rows are hard
        for s, rows in enumerate(force_hard):
            c["hard"][:, T0 + s] = False
            for b in rows:
                c["hard"][b, T0 + s] = True
    bf = lambda x: x.to(torch.bfloat16)
    dv = lambda x: x.to(device)
    cache = TaHDuoCache().enable_slabs(T0 + steps + 8, T0 + steps + 8)
    ocache = O.OracleCache()
    valid_all = c["valid"]
    pos_all = (torch.cumsum(valid_all, -1) - 1).clamp(min=0)
    tok = lambda x: x.transpose(1, 2)
    n_depth1_decode = 0

    def step(lo, hi):
        """Feed tokens [lo, hi) at depth 0, then their hard subset at depth 1, to both implementations."""
        nonlocal n_depth1_decode
        sl = slice(lo, hi)
        pos, valid, hard = pos_all[:, sl], valid_all[:, sl], c["hard"][:, sl]
        q1, k1, v1 = (bf(c[n][:, :, sl]) for n in ("q1", "k1", "v1"))
        # ours (device)
        m0 = build_attention_mask(dv(pos), dv(valid), cache, 0, torch.float32)
        cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, dv(pos), dv(valid)
        k, v = cache.update(dv(k1), dv(v1), 0)
        a1, _ = duo_attention_forward(_layer(), dv(q1), k, v, m0, scaling=c["scale"])
        pad, q2, k2, v2, pos2, val2 = gather_active(dv(hard), *(tok(dv(bf(c[n][:, :, sl]))) for n in ("q2", "k2", "v2")),
                                                    dv(pos), dv(valid))
        a2 = None
        if pad.shape[1]:
            m1 = build_attention_mask(pos2, val2, cache, 1, torch.float32)
            cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 1, pos2, val2
            k, v = cache.update(tok(k2), tok(v2), 0)
            a2, _ = duo_attention_forward(_layer(), tok(q2), k, v, m1, scaling=c["scale"])
        # reference formulation (host)
        r0 = O.build_attention_mask(pos, valid, ocache, 0, torch.float32)
        ocache.current_iter_depth, ocache.position_ids_to_cache, ocache.valid_mask_to_cache = 0, pos, valid
        K, V = ocache.update(k1.float(), v1.float(), 0)
        b1 = O.sdpa_dense(q1.float(), K, V, r0, c["scale"])
        rpad, rq2, rk2, rv2, rpos2, rval2 = O.gather_active(hard, *(tok(bf(c[n][:, :, sl]).float()) for n in ("q2", "k2", "v2")),
                                                            pos, valid)
        assert torch.equal(pad.cpu(), rpad)
        vb = valid.bool()
        np.testing.assert_allclose(a1.cpu()[vb].float().numpy(), b1[vb].numpy(), atol=2e-2, rtol=2e-2)
        if rpad.shape[1]:
            r1 = O.build_attention_mask(rpos2, rval2, ocache, 1, torch.float32)
            ocache.current_iter_depth, ocache.position_ids_to_cache, ocache.valid_mask_to_cache = 1, rpos2, rval2
            K, V = ocache.update(tok(rk2), tok(rv2), 0)
            b2 = O.sdpa_dense(tok(rq2), K, V, r1, c["scale"])
            np.testing.assert_allclose(a2.cpu()[~rpad].float().numpy(), b2[~rpad].numpy(), atol=2e-2, rtol=2e-2)
            assert (a2.cpu()[rpad] == 0).all()  # pad rows: zeros (the reference leaves an unused average of V there)
            if hi - lo == 1:
                n_depth1_decode += 1
                assert rpad.shape[1] == 1

    with torch.no_grad():
        step(0, T0)
        for s in range(steps):
            step(T0 + s, T0 + s + 1)
    s1 = cache.slabs(0, 0)
    assert s1.len.tolist() == valid_all.sum(1).tolist() and int(s1.overflow) == 0
    assert cache.slabs(0, 1).len.tolist() == (c["hard"] & valid_all.bool()).sum(1).tolist()
    # protocol lengths follow the reference's cache (pad rows of depth-1 writes count, causal_cache.py:162-186)
    assert cache.get_seq_length(0) == ocache.get_seq_length(0) == T0 + steps
    assert cache.get_cache_length(0, 1) == ocache.get_cache_length(0, 1)
    assert torch.equal(cache.get_valid_mask_upto_iter(0, 1).cpu(), ocache.get_valid_mask_upto_iter(0, 1))
    assert torch.equal(cache.get_position_id_upto_iter(0, 1).cpu(), ocache.get_position_id_upto_iter(0, 1))
    return cache, n_depth1_decode
