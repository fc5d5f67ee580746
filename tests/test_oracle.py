"""Pins the CPU oracle: brute force, closed forms, library special cases and the
agreement of its independent restatements.  No GPU."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import duo_oracle as O
from oracle import duo_ref as R
from tests.cases import dense_to_varlen, make_dense_case, make_varlen_case, varlen_args


def test_predicate_brute_force():
    for qp, qd, kp, kd, kv in itertools.product(range(4), range(2), range(4), range(2), range(2)):
        expect = (kp <= qp) and (kd <= qd) and kv == 1
        assert O.duo_visible(qp, qd, kp, kd, kv) == expect
    # equality on both axes is visible: a token's depth-1 query sees its own depth-0 and depth-1 key
    assert O.duo_visible(3, 1, 3, 0) and O.duo_visible(3, 1, 3, 1)
    # depth-0 queries never see depth-1 keys
    assert not O.duo_visible(5, 0, 0, 1)


def _mask_brute(qpos, qvalid, cache_meta, depth, neg):
    """(b, i, j) loops; cache_meta = list of (pos (B,L), valid (B,L), depth) in write order per depth."""
    B, T = qpos.shape
    cols = []
    for d in range(depth + 1):
        for pos, valid, dd in cache_meta:
            if dd == d:
                for j in range(pos.shape[1]):
                    cols.append((pos[:, j], valid[:, j], d))
    for j in range(T):
        cols.append((qpos[:, j], qvalid[:, j], depth))
    out = np.full((B, T, len(cols)), neg, dtype=np.float64)
    for b in range(B):
        for i in range(T):
            for j, (p, v, d) in enumerate(cols):
                if O.duo_visible(int(qpos[b, i]), depth, int(p[b]), d, int(v[b])):
                    out[b, i, j] = 0.0
    return out


def test_mask_matches_brute_force_with_cache_and_padding():
    g = torch.Generator().manual_seed(0)
    B, T = 3, 7
    valid = torch.ones(B, T, dtype=torch.long)
    valid[1, :2] = 0
    valid[2, :5] = 0
    pos = (torch.cumsum(valid, -1) - 1).clamp(min=0)
    cache = O.OracleCache()
    k = torch.zeros(B, 1, T, 2)
    m0 = O.build_attention_mask(pos, valid, cache, 0, torch.float32)
    neg = torch.finfo(torch.float32).min
    np.testing.assert_array_equal(m0[:, 0].numpy(), _mask_brute(pos, valid, [], 0, neg))
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, valid
    cache.update(k, k, 0)
    hard = (torch.rand(B, T, generator=g) < 0.5) & (valid == 1)
    pad, pos2, val2 = O.gather_active(hard, pos, valid)
    m1 = O.build_attention_mask(pos2, val2, cache, 1, torch.float32)
    np.testing.assert_array_equal(m1[:, 0].numpy(), _mask_brute(pos2, val2, [(pos, valid, 0)], 1, neg))
    # a later depth-0 step does not see the depth-1 slots already cached
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 1, pos2, val2
    cache.update(k[:, :, : pos2.shape[1]], k[:, :, : pos2.shape[1]], 0)
    newpos = pos[:, -1:] + 1
    one = torch.ones(B, 1, dtype=torch.long)
    m2 = O.build_attention_mask(newpos, one, cache, 0, torch.float32)
    assert m2.shape[-1] == T + 1
    np.testing.assert_array_equal(m2[:, 0].numpy(), _mask_brute(newpos, one, [(pos, valid, 0)], 0, neg))


def test_mask_reduces_to_causal_without_hard_tokens():
    T = 9
    pos = torch.arange(T)[None]
    m = O.build_attention_mask(pos, torch.ones(1, T, dtype=torch.long), O.OracleCache(), 0, torch.float32)
    tri = torch.tril(torch.ones(T, T, dtype=torch.bool))
    assert torch.equal(m[0, 0] == 0, tri)
    assert O.build_attention_mask(torch.zeros(1, 0, dtype=torch.long), torch.zeros(1, 0, dtype=torch.long),
                                  None, 0, torch.float32) is None


def test_all_hard_depth1_mask_is_two_causal_blocks():
    T = 6
    pos = torch.arange(T)[None]
    val = torch.ones(1, T, dtype=torch.long)
    cache = O.OracleCache()
    cache.current_iter_depth, cache.position_ids_to_cache, cache.valid_mask_to_cache = 0, pos, val
    cache.update(torch.zeros(1, 1, T, 2), torch.zeros(1, 1, T, 2), 0)
    m = O.build_attention_mask(pos, val, cache, 1, torch.float32)[0, 0] == 0
    tri = torch.tril(torch.ones(T, T, dtype=torch.bool))
    assert torch.equal(m, torch.cat([tri, tri], 1))


def test_cache_update_returns_depth_major_concatenation():
    cache = O.OracleCache()
    writes = []
    g = torch.Generator().manual_seed(1)
    for step, (depth, n) in enumerate([(0, 4), (1, 2), (0, 1), (1, 1), (0, 1)]):
        k = torch.randn(2, 3, n, 5, generator=g)
        cache.current_iter_depth = depth
        cache.position_ids_to_cache = torch.full((2, n), step)
        cache.valid_mask_to_cache = torch.ones(2, n, dtype=torch.long)
        K, V = cache.update(k, -k, 7)
        writes.append((depth, k))
        want = torch.cat([w for d in range(depth + 1) for (dd, w) in writes if dd == d], dim=-2)
        assert torch.equal(K, want) and torch.equal(V, -want)
        assert cache.get_cache_iter_index_upto_iter(7, depth).tolist() == [
            d for d in range(depth + 1) for (dd, w) in writes if dd == d for _ in range(w.shape[-2])]
    assert cache.get_seq_length(7) == 6 and cache.get_cache_length(7) == 9
    assert cache.get_kv_length_upto_iter(7, 1) == 9 and cache.get_cache_length(7, 1) == 3
    assert cache.get_position_id_upto_iter(7, 0).shape == (2, 6)
    assert cache.get_position_id_upto_iter(3, 1, init_batch_size=2).shape == (2, 0)
    assert not cache.has_layer(0) and cache.has_layer(7)
    with pytest.raises(AssertionError):
        cache.update(torch.zeros(3, 3, 1, 5), torch.zeros(3, 3, 1, 5), 7)


def test_repeat_kv_is_repeat_interleave():
    x = torch.randn(2, 4, 3, 5)
    assert torch.equal(O.repeat_kv(x, 2), torch.repeat_interleave(x, 2, dim=1))
    assert O.repeat_kv(x, 1) is x


def test_sdpa_dense_matches_torch_library():
    g = torch.Generator().manual_seed(2)
    q, k, v = (torch.randn(2, h, 33, 16, generator=g) for h in (4, 2, 2))
    scale = 16 ** -0.5
    mine = O.sdpa_dense(q, k, v, None, scale)
    kk, vv = (torch.repeat_interleave(t, 2, dim=1) for t in (k, v))
    lib = F.scaled_dot_product_attention(q, kk, vv, scale=scale).transpose(1, 2)
    torch.testing.assert_close(mine, lib, atol=2e-6, rtol=1e-5)
    pos = torch.arange(33)[None].expand(2, 33)
    m = O.build_attention_mask(pos, torch.ones(2, 33, dtype=torch.long), O.OracleCache(), 0, torch.float32)
    mine = O.sdpa_dense(q, k, v, m, scale)
    lib = F.scaled_dot_product_attention(q, kk, vv, is_causal=True, scale=scale).transpose(1, 2)
    torch.testing.assert_close(mine, lib, atol=2e-6, rtol=1e-5)
    lib = F.scaled_dot_product_attention(q, kk, vv, attn_mask=m, scale=scale).transpose(1, 2)
    torch.testing.assert_close(mine, lib, atol=2e-6, rtol=1e-5)


def test_finfo_min_equals_minus_inf_on_defined_rows():
    g = torch.Generator().manual_seed(3)
    q, k, v = (torch.randn(1, 2, 12, 8, generator=g) for _ in range(3))
    see = torch.tril(torch.ones(12, 12, dtype=torch.bool))
    a = O.sdpa_dense(q, k, v, torch.where(see, 0.0, torch.finfo(torch.float32).min)[None, None], 0.3)
    b = O.sdpa_dense(q, k, v, torch.where(see, 0.0, -float("inf"))[None, None], 0.3)
    assert torch.equal(a, b)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_pack_scatter_against_nonzero(seed):
    g = torch.Generator().manual_seed(seed)
    B, S = 4, 19
    mask = torch.rand(B, S, generator=g) < 0.3
    if seed == 2:
        mask[1] = False
    x = torch.randn(B, S, 3, generator=g)
    ids = torch.arange(B * S).view(B, S)
    pad, gx, gids, none = O.gather_active(mask, x, ids, None)
    assert none is None
    assert pad.shape[1] == int(mask.sum(1).max())
    # valid entries in row-major order == boolean-mask indexing
    assert torch.equal(gx[~pad], x[mask]) and torch.equal(gids[~pad], ids[mask])
    assert torch.equal(gx[pad], torch.zeros_like(gx[pad])) and (gids[pad] == 0).all()
    idx, cu = O.hard_index(mask)
    assert idx.tolist() == mask.nonzero()[:, 1].tolist()
    assert cu.tolist() == [0] + torch.cumsum(mask.sum(1), 0).tolist()
    ridx, rcu = R.hard_index(mask.numpy())
    assert ridx.tolist() == idx.tolist() and rcu.tolist() == cu.tolist()
    # scatter(gather(x)) restores active rows, leaves others untouched
    dest = torch.full_like(x, -7.0)
    back = O.scatter_back(mask, gx, dest)
    assert torch.equal(back[mask], x[mask]) and (back[~mask] == -7).all() and (dest == -7).all()
    amask = torch.rand(B, S, generator=g) < 0.5
    back2 = O.scatter_back(mask, gx, dest, assignment_mask=amask)
    assert torch.equal(back2[mask & amask], x[mask & amask]) and (back2[~(mask & amask)] == -7).all()
    assert O.scatter_back(mask, gx, dest, in_place=True) is dest


def test_gather_active_empty_mask():
    mask = torch.zeros(2, 5, dtype=torch.bool)
    pad, gx = O.gather_active(mask, torch.randn(2, 5, 3))
    assert pad.shape == (2, 0) and gx.shape == (2, 0, 3)


def _dense_vs_rows(c):
    v = dense_to_varlen(c)
    o1d, o2d, pad = O.duo_prefill_dense(c["q1"], c["k1"], c["v1"], c["q2"], c["k2"], c["v2"], c["hard"],
                                        c["scale"], valid_mask=c["valid"])
    o1, lse1, o2, lse2 = O.duo_rows_f64(*varlen_args(v))
    valid = c["valid"].bool()
    np.testing.assert_allclose(o1d[valid].numpy(), o1, atol=2e-5, rtol=1e-4)
    np.testing.assert_allclose(o2d[~pad].numpy(), o2, atol=2e-5, rtol=1e-4)
    return v, (o1, lse1, o2, lse2)


def test_dense_formulation_matches_row_loops():
    c = make_dense_case(5, B=2, T=40, p_hard=0.2, Hq=4, Hkv=2, D=16)
    _dense_vs_rows(c)


def test_dense_formulation_matches_row_loops_left_padded():
    c = make_dense_case(6, B=3, T=24, p_hard=0.3, Hq=2, Hkv=1, D=8, left_pad=[0, 5, 17])
    _dense_vs_rows(c)


def test_c_oracle_matches_row_loops():
    v = make_varlen_case(7, [37, 5, 64], 0.15, Hq=4, Hkv=2, D=32)
    a = O.duo_rows_f64(*varlen_args(v))
    b = R.fwd(*varlen_args(v))
    for x, y in zip(a, b):
        np.testing.assert_allclose(x, y, atol=2e-6, rtol=1e-5)


def test_c_oracle_with_cache_prefix_and_extra_depth1_keys():
    v = make_varlen_case(8, [3, 1, 9], 0.5, Hq=2, Hkv=2, D=16, seqlens_k=[10, 6, 9], extra_k2=3)
    assert len(v["pos_k2"]) > len(v["pos_q2"])
    a = O.duo_rows_f64(*varlen_args(v))
    b = R.fwd(*varlen_args(v))
    for x, y in zip(a, b):
        np.testing.assert_allclose(x, y, atol=2e-6, rtol=1e-5)
    o1t, o2t = O.duo_varlen_torch(*[t.double() if torch.is_tensor(t) else t for t in varlen_args(v)])
    np.testing.assert_allclose(o1t.numpy(), a[0], atol=1e-9)
    np.testing.assert_allclose(o2t.numpy(), a[2], atol=1e-9)


def test_no_hard_tokens_is_plain_causal_sdpa():
    v = make_varlen_case(9, [33], 0.0, Hq=4, Hkv=2, D=16)
    assert len(v["pos_q2"]) == 0
    o1 = R.fwd(*varlen_args(v))[0]
    q, k, vv = (v[n].transpose(0, 1)[None] for n in ("q1", "k1", "v1"))
    lib = F.scaled_dot_product_attention(q, O.repeat_kv(k, 2), O.repeat_kv(vv, 2), is_causal=True, scale=v["scale"])
    np.testing.assert_allclose(o1, lib[0].transpose(0, 1).numpy(), atol=2e-6, rtol=1e-5)


def test_lse_is_log_partition():
    v = make_varlen_case(10, [12], 0.4, Hq=1, Hkv=1, D=8)
    o1, lse1, o2, lse2 = R.fwd(*varlen_args(v))
    q, k = v["q1"][:, 0].double(), v["k1"][:, 0].double()
    s = (q @ k.T) * v["scale"]
    s = s.masked_fill(~torch.tril(torch.ones(12, 12, dtype=torch.bool)), -float("inf"))
    np.testing.assert_allclose(lse1[0], torch.logsumexp(s, -1).numpy(), atol=1e-5)


def _grads_torch(v, do1, do2):
    t = {k: (x.double().requires_grad_(True) if torch.is_tensor(x) and x.is_floating_point() else x)
         for k, x in v.items()}
    o1, o2 = O.duo_varlen_torch(*varlen_args(t))
    ((o1 * do1.double()).sum() + (o2 * do2.double()).sum()).backward()
    z = lambda x: x.grad if x.grad is not None else torch.zeros_like(x)
    return [z(t[n]).numpy() for n in ("q1", "k1", "v1", "q2", "k2", "v2")]


def test_backward_autograd_matches_analytic_c():
    v = make_varlen_case(11, [21, 8], 0.3, Hq=4, Hkv=2, D=16, seqlens_k=[21, 12], extra_k2=2)
    g = torch.Generator().manual_seed(12)
    do1, do2 = torch.randn(v["q1"].shape, generator=g), torch.randn(v["q2"].shape, generator=g)
    ga = _grads_torch(v, do1, do2)
    gc = R.bwd(*varlen_args(v), do1.numpy(), do2.numpy())
    for a, c in zip(ga, gc):
        np.testing.assert_allclose(a, c, atol=3e-6, rtol=1e-4)


def test_backward_finite_differences():
    v = make_varlen_case(13, [6], 0.5, Hq=2, Hkv=1, D=4)
    assert len(v["pos_q2"]) >= 2
    g = torch.Generator().manual_seed(14)
    do1, do2 = torch.randn(v["q1"].shape, generator=g), torch.randn(v["q2"].shape, generator=g)
    grads = dict(zip(("q1", "k1", "v1", "q2", "k2", "v2"), _grads_torch(v, do1, do2)))

    def loss(case):
        o1, _, o2, _ = O.duo_rows_f64(*varlen_args(case))
        return float((o1 * do1.numpy()).sum() + (o2 * do2.numpy()).sum())

    eps = 1e-5
    rng = np.random.default_rng(0)
    for name in ("q1", "k1", "v1", "q2", "k2", "v2"):
        base = v[name].double().numpy()
        for _ in range(6):
            idx = tuple(rng.integers(0, s) for s in base.shape)
            hi, lo = base.copy(), base.copy()
            hi[idx] += eps
            lo[idx] -= eps
            fd = (loss({**v, name: torch.from_numpy(hi)}) - loss({**v, name: torch.from_numpy(lo)})) / (2 * eps)
            assert abs(fd - grads[name][idx]) < 1e-6 * max(1.0, abs(fd)), (name, idx, fd, grads[name][idx])


def test_depth0_kv_gradient_collects_both_streams():
    """dK1/dV1 = contribution of depth-0 queries + contribution of depth-1 queries (linearity in dO)."""
    v = make_varlen_case(15, [10], 0.5, Hq=2, Hkv=1, D=8)
    g = torch.Generator().manual_seed(16)
    do1, do2 = torch.randn(v["q1"].shape, generator=g).numpy(), torch.randn(v["q2"].shape, generator=g).numpy()
    both = R.bwd(*varlen_args(v), do1, do2)
    only1 = R.bwd(*varlen_args(v), do1, np.zeros_like(do2))
    only2 = R.bwd(*varlen_args(v), np.zeros_like(do1), do2)
    for a, b, c in zip(both, only1, only2):
        np.testing.assert_allclose(a, b + c, atol=1e-6)
    assert np.abs(only2[1]).max() > 0 and np.abs(only2[2]).max() > 0  # depth-1 queries reach dK1, dV1
    assert np.abs(only1[4]).max() == 0 and np.abs(only1[5]).max() == 0  # depth-0 queries never reach dK2, dV2
    assert np.abs(only2[0]).max() == 0  # dQ1 only from its own stream


def test_decode_row_equals_last_prefill_row():
    v = make_varlen_case(17, [9, 14], 0.4, Hq=4, Hkv=2, D=8)
    o1, lse1, o2, lse2 = O.duo_rows_f64(*varlen_args(v))
    last = [int(v["cu_q1"][b + 1]) - 1 for b in range(2)]
    qpos = [int(v["cu_q1"][b + 1] - v["cu_q1"][b]) - 1 for b in range(2)]
    od, lsed = O.duo_decode_f64(v["q1"][last], v["k1"], v["v1"], v["cu_k1"], v["k2"], v["v2"], v["pos_k2"],
                                v["cu_k2"], qpos, [0, 0], v["scale"])
    np.testing.assert_allclose(od, o1[last], atol=1e-12)
    np.testing.assert_allclose(lsed, lse1[:, last].T, atol=1e-12)
    # a depth-1 decode row equals the depth-1 prefill row of the same position
    for b in range(2):
        r = int(v["cu_q2"][b + 1]) - 1
        if r < int(v["cu_q2"][b]):
            continue
        p = int(v["pos_q2"][r])
        od, _ = O.duo_decode_f64(v["q2"][[r] * 2], v["k1"], v["v1"], v["cu_k1"], v["k2"], v["v2"], v["pos_k2"],
                                 v["cu_k2"], [p if bb == b else 0 for bb in range(2)], [1, 1], v["scale"])
        np.testing.assert_allclose(od[b], o2[r], atol=1e-12)


def test_visible_pairs_closed_form():
    v = make_varlen_case(18, [50, 7], 0.2, Hq=2, Hkv=1, D=4, seqlens_k=[60, 7], extra_k2=4)
    n = O.visible_pairs(v["cu_q1"], v["cu_k1"], v["pos_q2"], v["pos_k2"], v["cu_q2"], v["cu_k2"])
    brute = 0
    for b in range(2):
        lq, lk = v["cu_q1"][b + 1] - v["cu_q1"][b], v["cu_k1"][b + 1] - v["cu_k1"][b]
        for i in range(lq):
            brute += sum(O.duo_visible(i + lk - lq, 0, j, 0) for j in range(lk))
        for r in range(v["cu_q2"][b], v["cu_q2"][b + 1]):
            brute += sum(O.duo_visible(v["pos_q2"][r], 1, j, 0) for j in range(lk))
            brute += sum(O.duo_visible(v["pos_q2"][r], 1, v["pos_k2"][j], 1)
                         for j in range(v["cu_k2"][b], v["cu_k2"][b + 1]))
    assert n == brute
    # single full sequence, no prefix: L(L+1)/2 + sum(pos+1) + n2(n2+1)/2
    w = make_varlen_case(19, [100], 0.1, Hq=1, Hkv=1, D=4)
    n2 = len(w["pos_q2"])
    want = 100 * 101 // 2 + int((w["pos_q2"] + 1).sum()) + n2 * (n2 + 1) // 2
    assert O.visible_pairs(w["cu_q1"], w["cu_k1"], w["pos_q2"], w["pos_k2"], w["cu_q2"], w["cu_k2"]) == want
