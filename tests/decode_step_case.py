"""One generation step's attention, fused (tah_duo_decode_step) against the two calls it replaces (tah_qk_prep with
append + tah_duo_decode): cache contents, positions and lengths have to agree bit for bit; the outputs as well, up to
the last bit of a rare element (same arithmetic in the same order, but two kernels: the compiler may contract a
multiply and an add into one instruction in one of them and not in the other)."""
import copy

import torch

BF = torch.bfloat16


def _slabs(B, cap, hkv, lens, with_pos, g, dev):
    from tah_amd.kv_cache import KvSlabs
    s = KvSlabs(B, cap, hkv, 128, with_pos=with_pos, device=dev)
    s.k.copy_(torch.randn(s.k.shape, generator=g).to(BF))
    s.v.copy_(torch.randn(s.v.shape, generator=g).to(BF))
    s.len.copy_(torch.tensor(lens, dtype=torch.int32))
    return s


def run(dev, *, B, hq, hkv, seed=0, max_len=90, hidden=256, cap1=128, cap2=64, full_slab=False):
    """full_slab: the depth-0 slabs hold exactly the longest sequence, so that sequence's new row does not fit: both
    paths have to raise the overflow flag, leave slab and length alone and attend over what is cached."""
    from tah_amd import kv_cache
    g = torch.Generator().manual_seed(seed)
    lens1 = torch.randint(1, max_len, (B,), generator=g).tolist()
    if full_slab:
        lens1[1] = max(lens1) + 1   # one longest sequence, active
        cap1 = lens1[1]
    lens2 = [int(torch.randint(0, min(l, cap2 - 1) + 1, (1,), generator=g)) for l in lens1]
    c1 = _slabs(B, cap1, hkv, lens1, False, g, dev)
    c2 = _slabs(B, cap2, hkv, lens2, True, g, dev)
    for b in range(B):  # depth-1 rows sit at increasing positions below the sequence's length
        c2.pos[b, :lens2[b]] = torch.sort(torch.randperm(lens1[b], generator=g)[:lens2[b]]).values.to(torch.int32)
    rn = lambda *s: torch.randn(*s, generator=g).to(BF).to(dev)
    q, k, v = rn(B, hq, 128) * 3, rn(B, hkv, 128) * 3, rn(B, hkv, 128)
    qw, kw = (1 + 0.1 * torch.randn(128, generator=g)).to(BF).to(dev), (1 + 0.1 * torch.randn(128, generator=g)).to(BF).to(dev)
    x = rn(B, hidden) * 2
    rows = torch.arange(B, dtype=torch.int32, device=dev)
    cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
    pos = torch.tensor(lens1, dtype=torch.int32, device=dev)
    ang = torch.randn(B, 128, generator=g)
    cos, sin = ang.cos().to(BF).to(dev), ang.sin().to(BF).to(dev)
    active = torch.ones(B, dtype=torch.bool)
    active[B // 3] = False        # a finished row: not cached, sees nothing
    hard = torch.rand(B, generator=g) < 0.4
    hard[0], hard[B // 3] = True, False
    active, hard = active.to(dev), hard.to(dev)
    minus1 = torch.full((B,), -1, dtype=torch.int32, device=dev)
    scale = 128 ** -0.5
    results = {}
    for depth in (0, 1):
        sel = active if depth == 0 else hard
        slot_of = torch.where(sel, rows, minus1)
        q_pos = torch.where(sel, pos, minus1)
        q_depth = torch.zeros(B, dtype=torch.int32, device=dev) if depth == 0 else hard.to(torch.int32)
        out = []
        for fused in (False, True):
            a1, a2 = copy.deepcopy(c1), copy.deepcopy(c2)
            tgt = a1 if depth == 0 else a2
            packed = torch.zeros(32 * hq * 128, dtype=BF, device=dev) if B <= 32 else None
            common = dict(cache=tgt, cu_new=cu, slot_of=slot_of, pos_new=pos if depth == 1 else None, norm_input=x, norm_eps=1e-6)
            if fused:
                o = kv_cache.decode_step(q, k, v, qw, kw, cos, sin, 1e-6, append_at=tgt.len.clone(), q_slot=rows, q_pos=q_pos,
                                         c1=a1, c2=a2, scale=scale, q_depth=q_depth, out_packed=packed, **common)
            else:
                qo, _ = kv_cache.qk_norm_rope(q, k, qw, kw, cos, sin, 1e-6, v=v, one_row_per_seq=True, **common)
                o = kv_cache.decode(qo, rows, q_pos, a1, a2, scale=scale, q_depth=q_depth, out_packed=packed)
            out.append((o, packed, a1, a2))
        (oa, pa, a1, a2), (ob, pb, b1, b2) = out
        assert torch.allclose(oa.float(), ob.float(), rtol=2.0 ** -7, atol=2.0 ** -12), f"depth {depth}: outputs differ"
        assert (oa != ob).float().mean() < 1e-3, f"depth {depth}: more than a rare last bit differs"
        from tests.test_linear_rows import unpack_rows
        assert pb is None or torch.equal(unpack_rows(pb.cpu(), hq * 128)[:B], ob.cpu().reshape(B, -1))
        for sa, sb in ((a1, b1), (a2, b2)):
            assert torch.equal(sa.k, sb.k) and torch.equal(sa.v, sb.v) and torch.equal(sa.len, sb.len)
        over = 1 if (full_slab and depth == 0) else 0
        assert int(a1.overflow) == int(b1.overflow) == over and int(a2.overflow) == int(b2.overflow) == 0
        assert torch.equal(a2.pos, b2.pos)
        tgt_a, src = (a1, c1) if depth == 0 else (a2, c2)
        grew = sel.cpu().to(torch.int32)
        if over:
            grew[1] = 0   # the row that did not fit
        assert torch.equal(tgt_a.len.cpu(), src.len.cpu() + grew)  # the step did append
        assert oa[B // 3].abs().max() == 0                                              # the finished row saw nothing
        results[depth] = oa
    if not full_slab:  # a row told to append below its slab's end: the step reports it (flag value 2)
        a1, a2 = copy.deepcopy(c1), copy.deepcopy(c2)
        at = a1.len.clone()
        victim = next(b for b in range(B) if bool(active[b]) and lens1[b] >= 2)
        at[victim] -= 1
        kv_cache.decode_step(q, k, v, qw, kw, cos, sin, 1e-6, append_at=at, q_slot=rows, q_pos=torch.where(active, pos, minus1),
                             c1=a1, c2=a2, scale=scale, q_depth=torch.zeros(B, dtype=torch.int32, device=dev), cache=a1, cu_new=cu,
                             slot_of=torch.where(active, rows, minus1), pos_new=None, norm_input=x, norm_eps=1e-6)
        assert int(a1.overflow) == 2 and int(a1.len[victim]) == lens1[victim]
    return results


def run_mixed(dev, *, B, hq, hkv, seed=0, max_len=90, hidden=256, cap1=128, cap2=64):
    """Rows at different latent iterations in one call (append_depth): rows at depth 0 append to the depth-0 slabs and
    see them, rows at depth 1 append to the depth-1 slabs (with their position) and see both.  Against two tah_qk_prep
    calls, one per depth with the other depth's rows masked out, followed by one tah_duo_decode."""
    from tah_amd import kv_cache
    g = torch.Generator().manual_seed(seed)
    lens1 = torch.randint(2, max_len, (B,), generator=g).tolist()
    lens2 = [int(torch.randint(0, min(l, cap2 - 1), (1,), generator=g)) for l in lens1]
    c1 = _slabs(B, cap1, hkv, lens1, False, g, dev)
    c2 = _slabs(B, cap2, hkv, lens2, True, g, dev)
    for b in range(B):
        c2.pos[b, :lens2[b]] = torch.sort(torch.randperm(lens1[b] - 1, generator=g)[:lens2[b]]).values.to(torch.int32)
    rn = lambda *s: torch.randn(*s, generator=g).to(BF).to(dev)
    q, k, v = rn(B, hq, 128) * 3, rn(B, hkv, 128) * 3, rn(B, hkv, 128)
    qw, kw = (1 + 0.1 * torch.randn(128, generator=g)).to(BF).to(dev), (1 + 0.1 * torch.randn(128, generator=g)).to(BF).to(dev)
    x = rn(B, hidden) * 2
    rows = torch.arange(B, dtype=torch.int32, device=dev)
    cu = torch.arange(B + 1, dtype=torch.int32, device=dev)
    ang = torch.randn(B, 128, generator=g)
    cos, sin = ang.cos().to(BF).to(dev), ang.sin().to(BF).to(dev)
    active = torch.ones(B, dtype=torch.bool)
    active[B // 3] = False
    depth = (torch.rand(B, generator=g) < 0.5)
    depth[0], depth[1] = True, False
    active, depth = active.to(dev), depth.to(dev)
    minus1 = torch.full((B,), -1, dtype=torch.int32, device=dev)
    # a row at depth 1 has its depth-0 K/V in the slabs already: its position is the last cached one
    pos = torch.tensor(lens1, dtype=torch.int32, device=dev) - depth.to(torch.int32)
    q_pos = torch.where(active, pos, minus1)
    q_depth = depth.to(torch.int32)
    slot_all = torch.where(active, rows, minus1)
    scale = 128 ** -0.5
    a1, a2 = copy.deepcopy(c1), copy.deepcopy(c2)
    common = dict(cu_new=cu, norm_input=x, norm_eps=1e-6)
    qo, _ = kv_cache.qk_norm_rope(q, k, qw, kw, cos, sin, 1e-6, v=v, one_row_per_seq=True, cache=a1,
                                  slot_of=torch.where(active & ~depth, rows, minus1), **common)
    kv_cache.qk_norm_rope(q, k, qw, kw, cos, sin, 1e-6, v=v, one_row_per_seq=True, cache=a2, pos_new=pos,
                          slot_of=torch.where(active & depth, rows, minus1), **common)
    oa = kv_cache.decode(qo, rows, q_pos, a1, a2, scale=scale, q_depth=q_depth)
    b1, b2 = copy.deepcopy(c1), copy.deepcopy(c2)
    append_at = torch.where(depth, b2.len, b1.len)
    ob = kv_cache.decode_step(q, k, v, qw, kw, cos, sin, 1e-6, cache=b2, append_at=append_at, append_depth=q_depth, q_slot=rows,
                              q_pos=q_pos, c1=b1, c2=b2, scale=scale, slot_of=slot_all, pos_new=pos, q_depth=q_depth, **common)
    assert torch.allclose(oa.float(), ob.float(), rtol=2.0 ** -7, atol=2.0 ** -12) and (oa != ob).float().mean() < 1e-3
    for sa, sb in ((a1, b1), (a2, b2)):
        assert torch.equal(sa.k, sb.k) and torch.equal(sa.v, sb.v) and torch.equal(sa.len, sb.len) and int(sa.overflow) == int(sb.overflow) == 0
    assert torch.equal(a2.pos, b2.pos)
    assert torch.equal(b1.len.cpu(), c1.len.cpu() + (active & ~depth).cpu().to(torch.int32))
    assert torch.equal(b2.len.cpu(), c2.len.cpu() + (active & depth).cpu().to(torch.int32))
