"""Launch-order table (tah_duo_schedule_build): it lists every tile exactly once, heaviest first, and using
it changes no result.  The CPU tests run the kernels on the CPU execution shim; the GPU tests call the library."""
import numpy as np
import pytest
import torch

from tests import emu_util
from tests.cases import make_varlen_case, varlen_args

HEADER = 16
MAGIC = 0x54414853


def _to_dev(case, device="cpu"):
    out = {}
    for k, v in case.items():
        if isinstance(v, np.ndarray):
            out[k] = torch.from_numpy(v.copy()).to(device)
        elif torch.is_tensor(v):
            out[k] = v.to(torch.bfloat16).to(device)
        else:
            out[k] = v
    return out


def _schedule(ops, dev, hq, hkv):
    return ops.duo_schedule(dev["cu_q1"], dev["cu_k1"], dev["cu_q2"], dev["cu_k2"], dev["pos_q2"], hq, hkv,
                            dev["q1"].shape[0], dev["k1"].shape[0], dev["k2"].shape[0])


def _tiles_in_order(cu_a, cu_b, tile):
    """(stream, sequence, first row) of every tile in the order the kernels count them: the depth-0 stream's tiles
    sequence by sequence, then the depth-1 stream's."""
    out = []
    for second, cu in ((0, cu_a), (1, cu_b)):
        for b in range(len(cu) - 1):
            for r in range(int(cu[b]), int(cu[b + 1]), tile):
                out.append((second, b, r))
    return out


def _expected_tiles(cu_a, cu_b, tile):
    want = set()
    for second, cu in ((0, cu_a), (1, cu_b)):
        for b in range(len(cu) - 1):
            for r in range(int(cu[b]), int(cu[b + 1]), tile):
                want.add((second, b, r))
    return want


def _visible_pairs_q(case, second, b, r0, tile):
    """(query row, key) pairs a query tile has to look at, counted straight from the visibility rule."""
    cu_q1, cu_k1, cu_q2, cu_k2 = (case[k] for k in ("cu_q1", "cu_k1", "cu_q2", "cu_k2"))
    lq1, lk1 = cu_q1[b + 1] - cu_q1[b], cu_k1[b + 1] - cu_k1[b]
    if not second:
        rows = range(r0, min(r0 + tile, cu_q1[b + 1]))
        return max((r - cu_q1[b]) + (lk1 - lq1) + 1 for r in rows)  # keys the last row sees
    rows = range(r0, min(r0 + tile, cu_q2[b + 1]))
    return max(min(int(case["pos_q2"][r]) + 1, lk1) for r in rows) + (cu_k2[b + 1] - cu_k2[b])


def _check_table(table, case, hq, hkv):
    t = table.cpu().numpy()
    g = hq // hkv
    bm = 32 * (8 // g)
    nseq = len(case["cu_q1"]) - 1
    assert t[0] == MAGIC and t[1] == nseq and t[2] == g
    assert (t[3], t[4], t[5], t[6]) == (case["q1"].shape[0], case["q2"].shape[0], case["k1"].shape[0], case["k2"].shape[0])
    nq, nk = int(t[7]), int(t[8])
    assert len(t) == HEADER + 2 * (nq + nk)
    for lst, n, tile, cu_a, cu_b in ((t[HEADER:HEADER + 2 * nq], nq, bm, case["cu_q1"], case["cu_q2"]),
                                     (t[HEADER + 2 * nq:], nk, 128, case["cu_k1"], case["cu_k2"])):
        x, y = lst[0::2], lst[1::2]
        tiles = _tiles_in_order(cu_a, cu_b, tile)
        # a permutation of the tile numbers 0 .. n-1: whatever the boundaries, every tile is visited once
        assert sorted(x.tolist()) == list(range(n)) and not y.any()
        used = x < len(tiles)
        n_used = int(used.sum())
        assert n_used == len(tiles) and used[:n_used].all()  # numbers without a tile come last
        got = [tiles[int(v)] for v in x[:n_used]]
        assert len(set(got)) == len(got) and set(got) == _expected_tiles(cu_a, cu_b, tile)
    # query tiles: the keys a tile has to walk over never grow along the list (in 64-key steps)
    tiles = _tiles_in_order(case["cu_q1"], case["cu_q2"], bm)
    steps = [-(-_visible_pairs_q(case, *tiles[int(v)], bm) // 64) for v in t[HEADER:HEADER + 2 * nq:2] if v < len(tiles)]
    # a depth-1 tile also walks every 64-key tile of its depth-1 segment, which rounds up separately from the
    # depth-0 part: allow one step of slack against the straight count
    assert all(a >= b - 1 for a, b in zip(steps, steps[1:])), steps


CASES = [
    (2, 1, [70, 300, 5, 129], 0.3, None),
    (4, 2, [64, 0, 200, 31], 0.2, None),         # an empty sequence in the middle
    (2, 1, [40, 90, 17], 0.25, [100, 90, 80]),   # cached prefixes: more keys than queries
    (8, 1, [33, 150], 0.0, None),                # no depth-1 rows at all
]


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
@pytest.mark.parametrize("hq,hkv,seqlens,p,seqlens_k", CASES)
def test_schedule_lists_every_tile_once_heaviest_first(hq, hkv, seqlens, p, seqlens_k):
    from tah_amd import ops
    case = make_varlen_case(7 + hq, seqlens, p, Hq=hq, Hkv=hkv, D=128, seqlens_k=seqlens_k, extra_k2=3 if seqlens_k else 0)
    dev = _to_dev(case)
    with emu_util.emulated():
        table = _schedule(ops, dev, hq, hkv)
    _check_table(table, case, hq, hkv)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
@pytest.mark.parametrize("hq,hkv,seqlens,p,seqlens_k", [(2, 1, [70, 5, 140], 0.3, None), CASES[2]])
def test_forward_and_backward_do_not_depend_on_the_schedule(hq, hkv, seqlens, p, seqlens_k):
    from tah_amd import ops
    case = make_varlen_case(11 + hq, seqlens, p, Hq=hq, Hkv=hkv, D=128, seqlens_k=seqlens_k, extra_k2=3 if seqlens_k else 0)
    dev = _to_dev(case)
    g = torch.Generator().manual_seed(5)
    do1 = torch.randn(dev["q1"].shape, generator=g).to(torch.bfloat16)
    do2 = torch.randn(dev["q2"].shape, generator=g).to(torch.bfloat16)
    with emu_util.emulated():
        table = _schedule(ops, dev, hq, hkv)
        plain = ops.duo_fwd_varlen(*varlen_args(dev))
        listed = ops.duo_fwd_varlen(*varlen_args(dev), schedule=table)
        for a, b in zip(plain, listed):
            assert torch.equal(a, b)
        o1, lse1, o2, lse2 = plain
        bwd = lambda s: ops.duo_bwd_varlen(dev["q1"], dev["k1"], dev["v1"], o1, lse1, do1, dev["cu_q1"], dev["cu_k1"], dev["q2"],
                                           dev["k2"], dev["v2"], o2, lse2, do2, dev["pos_q2"], dev["pos_k2"], dev["cu_q2"],
                                           dev["cu_k2"], dev["scale"], schedule=s)
        for a, b in zip(bwd(None), bwd(table)):
            assert torch.equal(a, b)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_a_table_built_for_other_sizes_is_ignored():
    from tah_amd import ops
    dev_a = _to_dev(make_varlen_case(3, [70, 200], 0.3, Hq=2, Hkv=1, D=128))
    dev_b = _to_dev(make_varlen_case(4, [150, 66], 0.3, Hq=2, Hkv=1, D=128))
    with emu_util.emulated():
        table_a = _schedule(ops, dev_a, 2, 1)
        plain = ops.duo_fwd_varlen(*varlen_args(dev_b))
        stale = ops.duo_fwd_varlen(*varlen_args(dev_b), schedule=table_a)
    for a, b in zip(plain, stale):
        assert torch.equal(a, b)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_a_table_built_for_other_boundaries_of_the_same_sizes_changes_no_result():
    """Packed training: the same number of tokens every step, new document boundaries.  A table from another step has
    the call's sizes and is taken; being a permutation of the tile numbers it still makes the kernels visit every tile
    of the call's own boundaries once (also when these have more tiles than the table's had)."""
    from tah_amd import ops
    mk = lambda seed, lens: _to_dev(make_varlen_case(seed, lens, 0.0, Hq=2, Hkv=1, D=128))
    dev_a, dev_b = mk(3, [256, 128, 128]), mk(4, [100, 130, 282])   # 512 rows each: 4 query tiles against 5
    g = torch.Generator().manual_seed(5)
    do1 = torch.randn(dev_b["q1"].shape, generator=g).to(torch.bfloat16)
    with emu_util.emulated():
        table_a = _schedule(ops, dev_a, 2, 1)
        assert table_a is not None
        plain = ops.duo_fwd_varlen(*varlen_args(dev_b))
        stale = ops.duo_fwd_varlen(*varlen_args(dev_b), schedule=table_a)
        for a, b in zip(plain, stale):
            assert torch.equal(a, b)
        o1, lse1, o2, lse2 = plain
        bwd = lambda s, ws: ops.duo_bwd_varlen(dev_b["q1"], dev_b["k1"], dev_b["v1"], o1, lse1, do1, dev_b["cu_q1"], dev_b["cu_k1"],
                                               dev_b["q2"], dev_b["k2"], dev_b["v2"], o2, lse2, do1[:0], dev_b["pos_q2"], dev_b["pos_k2"],
                                               dev_b["cu_q2"], dev_b["cu_k2"], dev_b["scale"], schedule=s, ds_workspace=ws)
        for ws in (None, False):
            for a, b in zip(bwd(None, ws), bwd(table_a, ws)):
                assert torch.equal(a, b)


@pytest.mark.skipif(not emu_util.have_host_clang(), reason="host clang++ not available")
def test_one_sequence_needs_no_table():
    from tah_amd import ops
    dev = _to_dev(make_varlen_case(3, [300], 0.3, Hq=2, Hkv=1, D=128))
    with emu_util.emulated():
        assert _schedule(ops, dev, 2, 1) is None


@pytest.mark.gpu
@pytest.mark.parametrize("seqlens,p", [([1397, 3210, 2561, 1024], 0.10), ([300, 0, 4096, 77, 1], 0.06)])
def test_gpu_schedule_table_and_results(seqlens, p):
    from tah_amd import ops
    case = make_varlen_case(21, seqlens, p)
    dev = _to_dev(case, "cuda")
    table = _schedule(ops, dev, 16, 8)
    _check_table(table, case, 16, 8)
    g = torch.Generator().manual_seed(5)
    do1 = torch.randn(dev["q1"].shape, generator=g).to(torch.bfloat16).cuda()
    do2 = torch.randn(dev["q2"].shape, generator=g).to(torch.bfloat16).cuda()
    plain = ops.duo_fwd_varlen(*varlen_args(dev))
    listed = ops.duo_fwd_varlen(*varlen_args(dev), schedule=table)
    for a, b in zip(plain, listed):
        assert torch.equal(a, b)
    o1, lse1, o2, lse2 = plain
    bwd = lambda s: ops.duo_bwd_varlen(dev["q1"], dev["k1"], dev["v1"], o1, lse1, do1, dev["cu_q1"], dev["cu_k1"], dev["q2"],
                                       dev["k2"], dev["v2"], o2, lse2, do2, dev["pos_q2"], dev["pos_k2"], dev["cu_q2"],
                                       dev["cu_k2"], dev["scale"], schedule=s)
    for a, b in zip(bwd(None), bwd(table)):
        assert torch.equal(a, b)
