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

``qk_prep_backward`` is the analytic gradient of the same two steps (no intermediate rounding), float64; pinned in the
same file against autograd through the installed transformers modules run in float64 and against finite differences.
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


def qk_prep_backward(q, k, q_weight, k_weight, cos, sin, eps, dq_out, dk_out):
    """Gradients of ``qk_prep`` (taken as the real-valued function: RMSNorm, weight, rotation): float64
    ``(dq, dk, dq_weight, dk_weight)`` for output gradients ``dq_out`` [rows, Hq, D], ``dk_out`` [rows, Hkv, D].

    With y = w * xh, xh = x * rs, rs = (mean(x^2) + eps)^(-1/2) and out = y cos + rotate_half(y) sin:
    dy = g cos + rotate_half^T(g sin) where rotate_half^T(u) = cat(u[64:], -u[:64]); dw = sum dy * xh;
    dx = rs * (dy w - xh * mean(dy w xh))."""
    c, s = cos[:, None, :].astype(np.float64), sin[:, None, :].astype(np.float64)

    def one(x, w, g):
        x, w, g = x.astype(np.float64), w.astype(np.float64), g.astype(np.float64)
        half = x.shape[-1] // 2
        rs = 1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
        xh = x * rs
        u = g * s
        dy = g * c + np.concatenate([u[..., half:], -u[..., :half]], axis=-1)
        dxh = dy * w
        dx = rs * (dxh - xh * np.mean(dxh * xh, axis=-1, keepdims=True))
        return dx, (dy * xh).sum(axis=(0, 1))

    dq, dqw = one(q, q_weight, dq_out)
    dk, dkw = one(k, k_weight, dk_out)
    return dq, dk, dqw, dkw
