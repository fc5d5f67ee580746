"""Seeded inputs for the top-k softmax mix (tah_model.py:57-75): bf16-representable logits and embeddings."""
import numpy as np
import torch

from oracle.topk_mix_ref import bf16_round


def make_case(seed, rows, V, H, *, distinct=False, scale=3.0, ties=0.0):
    g = np.random.default_rng(seed)
    if distinct:
        # every logit of a row a different bf16 value: a permutation of V distinct finite bf16 numbers
        # (the 4610 bf16 numbers with 2^-15 <= |x| <= 8, by bit pattern)
        pos = (np.arange(0x3800, 0x4101, dtype=np.uint32) << 16).view(np.float32)
        base = np.concatenate([-pos, pos])
        assert base.size >= V
        logits = np.stack([g.permutation(base)[:V] for _ in range(rows)]).astype(np.float32)
    else:
        logits = bf16_round((g.standard_normal((rows, V)) * scale).astype(np.float32))
        if ties:  # a plateau of equal values around the k-th place
            for r in range(rows):
                idx = g.choice(V, int(V * ties), replace=False)
                logits[r, idx] = np.sort(logits[r])[::-1][min(90, V - 1)]
    emb = bf16_round(g.standard_normal((V, H)).astype(np.float32))
    return logits, emb


def to_torch(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).to(device)
