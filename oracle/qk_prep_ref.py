"""CPU restatement of the step before the attention call: per-head RMSNorm of q and k, then the
rotary embedding.  TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py, never by the product.

The arithmetic lives in a third-party dependency of the reference that is not part of its tree:
``transformers`` (pinned 4.52.4 in the reference's pyproject.toml:21), called from the reference at
tah/model/tah_model.py:616-623 (the base model call whose layers run it).  Restated from its
published source:

* ``Qwen3RMSNorm.forward`` (transformers/models/qwen3/modeling_qwen3.py): in float32,
  ``x * rsqrt(mean(x^2) + eps)``, cast back to the input dtype, then ``weight * that`` in the input dtype;
* ``apply_rotary_pos_emb`` / ``rotate_half`` (same file): ``x * cos + cat(-x[64:], x[:64]) * sin``, every
  product and the sum rounded to the input dtype (bf16 eager arithmetic).

Pinned in tests/test_oracle_qk_prep.py against the installed transformers' own ``Qwen3RMSNorm`` and
``apply_rotary_pos_emb`` run on the CPU in bf16 (bit-exact up to the last-place effect of the
float32 summation order in the mean), and by what the mathematics fixes: unit weights give rows of
RMS 1 before the rotation, the rotation keeps the norm of every (i, i + 64) pair up to rounding,
position 0 (cos = 1, sin = 0) is the identity.
"""
import numpy as np


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 values rounded to the nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    r = ((u + bias) & np.uint32(0xFFFF0000)).view(np.float32)
    return np.where(np.isnan(x), x, r).astype(np.float32)


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """Qwen3RMSNorm.forward on bf16 data held as float32: x [..., D], w [D]."""
    x = x.astype(np.float32)
    var = np.mean(x * x, axis=-1, keepdims=True, dtype=np.float32)
    n = bf16_round(x * (np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)))
    return bf16_round(w.astype(np.float32) * n)


def rope(y: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """apply_rotary_pos_emb on one tensor: y [rows, H, D], cos / sin [rows, D] (bf16 values as float32)."""
    half = y.shape[-1] // 2
    rot = np.concatenate([-y[..., half:], y[..., :half]], axis=-1)
    c, s = cos[:, None, :].astype(np.float32), sin[:, None, :].astype(np.float32)
    return bf16_round(bf16_round(y * c) + bf16_round(rot * s))


def qk_prep(q, k, q_weight, k_weight, cos, sin, eps):
    """q [rows, Hq, D], k [rows, Hkv, D] -> (q_out, k_out), all bf16 values held as float32."""
    return rope(rms_norm(q, q_weight, eps), cos, sin), rope(rms_norm(k, k_weight, eps), cos, sin)


def rotary_tables(positions: np.ndarray, d: int = 128, theta: float = 1e6):
    """cos / sin [rows, D] as Qwen3RotaryEmbedding builds them (default rope type): float32 angles
    ``pos * theta^(-2i/D)``, duplicated over both halves, cos / sin cast to bf16."""
    inv = (1.0 / (theta ** (np.arange(0, d, 2, dtype=np.float32) / np.float32(d)))).astype(np.float32)
    f = positions.astype(np.float32)[:, None] * inv[None, :]
    emb = np.concatenate([f, f], axis=-1)
    return bf16_round(np.cos(emb).astype(np.float32)), bf16_round(np.sin(emb).astype(np.float32))
