"""Beam-search reorder of a cache with slabs: two caches filled alike (prefill at depth 0, the hard tokens again
at depth 1); one decodes a step as it is, the other is reordered first (row i continues row beam[i]) and decodes
the reordered inputs.  Row i of the second must equal row beam[i] of the first, at both depths."""
import types

import torch


def run(device, beam=(2, 0, 0), T0=12, seed=5):
    from tah_amd.attention import build_attention_mask, duo_attention_forward
    from tah_amd.cache import TaHDuoCache
    from tah_amd.pack import gather_active

    B, hq, hkv, D = len(beam), 2, 1, 128
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(device)
    layer = types.SimpleNamespace(num_key_value_groups=hq // hkv, layer_idx=0, training=False)
    scale = D ** -0.5
    pos = torch.arange(T0, device=device)[None].expand(B, T0).contiguous()
    valid = torch.ones(B, T0, dtype=torch.long, device=device)
    hard = (torch.rand(B, T0, generator=g) < 0.4).to(device)
    hard[:, 0] = True
    k1, v1 = rnd(B, hkv, T0, D), rnd(B, hkv, T0, D)
    k2, v2 = rnd(B, T0, hkv, D), rnd(B, T0, hkv, D)
    qn, kn, vn = rnd(B, hq, 1, D), rnd(B, hkv, 1, D), rnd(B, hkv, 1, D)       # the new token at depth 0
    qm, km, vm = rnd(B, hq, 1, D), rnd(B, hkv, 1, D), rnd(B, hkv, 1, D)       # ... and at depth 1 (every row hard)
    bidx = torch.tensor(beam, device=device)

    def filled():
        c = TaHDuoCache().enable_slabs(T0 + 4, T0 + 4)
        c.current_iter_depth, c.position_ids_to_cache, c.valid_mask_to_cache = 0, pos, valid
        c.update(k1, v1, 0)
        pad, k2p, v2p, pos2, val2 = gather_active(hard, k2, v2, pos, valid)
        val2 = val2 * (~pad).long()
        c.current_iter_depth, c.position_ids_to_cache, c.valid_mask_to_cache = 1, pos2, val2
        c.update(k2p.transpose(1, 2), v2p.transpose(1, 2), 0)
        return c

    def decode(c, sel):
        p1 = torch.full((B, 1), T0, dtype=torch.long, device=device)
        one = torch.ones(B, 1, dtype=torch.long, device=device)
        outs = []
        for depth, (q, k, v) in enumerate(((qn, kn, vn), (qm, km, vm))):
            c.current_iter_depth, c.position_ids_to_cache, c.valid_mask_to_cache = depth, p1, one
            mask = build_attention_mask(p1, one, c, depth)
            kk, vv = c.update(k[sel], v[sel], 0)
            o, _ = duo_attention_forward(layer, q[sel], kk, vv, mask, scaling=scale)
            outs.append(o.float().cpu())
        return outs

    with torch.no_grad():
        a = filled()
        plain = decode(a, torch.arange(B, device=device))
        b = filled()
        b.reorder_cache(bidx)
        lens0, lens1 = a.slabs(0, 0).len.cpu(), a.slabs(0, 1).len.cpu()
        moved = decode(b, bidx)
    assert b.slabs(0, 0).len.cpu().tolist() == lens0[list(beam)].tolist()
    assert b.slabs(0, 1).len.cpu().tolist() == lens1[list(beam)].tolist()
    return plain, moved, list(beam)
