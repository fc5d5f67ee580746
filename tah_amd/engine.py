"""Decode loop for a Think-at-Hard model on the native kernels.

The reference generates with ``TaHForCasualLM_generate`` (tah/model/utils.py:196-264): one
``TaHForCausalLM.forward`` per new token, each of which re-concatenates the KV cache per layer
(causal_cache.py:84-90), rebuilds a dense mask (tah_model.py:744-791), synchronises with the host several
times (tah_model.py:116, 580, 686, 705) and reads every sampled token back row by row (utils.py:243-245).
:class:`TaHDecodeEngine` runs the same computation -- the iteration loop of tah_model.py:580-706 for one
new token per sequence -- with

* per-(layer, depth) KV slabs preallocated for the whole generation (tah_amd.kv_cache.KvSlabs), appended
  in place by the fused q/k preparation kernel (``tah_qk_prep``) and read by the split-K decode kernel
  (``tah_duo_decode_static``: no allocation, so the step can be captured);
* a step of fixed shape: the second latent iteration runs for all B rows with the rows the decider did
  not select masked out (no K/V appended, no cache rows read, results dropped), so nothing in the step
  depends on a value the host would have to read -- no ``.item()``, no ``.any()``;
* batched sampling and end-of-sequence handling on the device;
* the whole step captured once in a HIP graph and replayed per token.

The linear layers of a decode step (at most 32 rows against weights of megabytes) run on weights re-ordered once
for streaming (``tah_linear_rows``: residual adds and the MLP's gate in their epilogues, rows handed from kernel to
kernel in the operand order of the matrix instruction); prefill, batches above 32 rows and the output head use torch
GEMMs (rocBLAS / hipBLASLt).  What is kept from the reference's forward loop, with the place it comes from:
depth-0 logits are the running sum (``additive_logits_update``, tah_model.py:78-83); the decider sees the
last hidden state (a two-layer MLP, hidden -> 512 -> 1, sigmoid, threshold -- the form the end-to-end
workload names; the reference's ``MLPIterDecider`` is a larger network over several layers,
iter_decider.py:193-301); hard rows get the top-k softmax mix of embedding rows as their next input
(``topk_softmax_input_update``, tah_model.py:57-75; here one ``tah_topk_mix`` launch) at the same position (tah_model.py:618), see the depth-0
and depth-1 caches, and their final logits are the sum of both iterations' logits.  LoRA adapters on the
second iteration (tah_model.py:581) are not modelled: both iterations use the same weights.
"""
from __future__ import annotations

import dataclasses
import math
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from . import ops
from ._capi import TahDuoError
from .kv_cache import KvSlabs, decode as _decode, decode_step as _decode_step, decode_step_supported, qk_norm_rope


@dataclasses.dataclass
class EngineConfig:
    """Qwen3-1.7B by default (the architecture of the end-to-end workload)."""
    hidden: int = 2048
    layers: int = 28
    hq: int = 16
    hkv: int = 8
    head_dim: int = 128
    intermediate: int = 6144
    vocab: int = 151936
    rms_eps: float = 1e-6
    rope_theta: float = 1e6
    decider_hidden: int = 512
    topk: int = 100


class Weights:
    """Plain tensors of a Qwen3-shaped decoder, the output head and the decider MLP (all bf16)."""

    def __init__(self, cfg: EngineConfig):
        self.cfg = cfg
        self.embed: torch.Tensor = None          # [V, H]
        self.lm_head: torch.Tensor = None        # [V, H] (the embedding itself when tied)
        self.norm: torch.Tensor = None           # [H]
        self.layers: List[dict] = []             # ln1, wqkv, qn, kn, wo, ln2, wgu, wdown
        self.dec_w1: torch.Tensor = None         # [Hd, H]
        self.dec_b1: torch.Tensor = None
        self.dec_w2: torch.Tensor = None         # [1, Hd]
        self.dec_b2: torch.Tensor = None
        self.threshold: float = 0.5
        self.norms_folded = False
        self.linear_packed = False
        self.lm_head_p: Optional[torch.Tensor] = None
        self.dec_w1_p: Optional[torch.Tensor] = None

    def fold_norms(self) -> "Weights":
        """Multiplies the input-norm weights into the projections that follow them (``wqkv *= ln1``, ``wgu *= ln2``,
        column-wise, rounded to the model dtype once).  What is left of the two RMSNorms of a layer is a factor per
        row, which ``tah_qk_prep`` and ``tah_silu_mul_normed`` apply: two launches per layer and latent iteration
        less.  Done once, in place."""
        if not self.norms_folded:
            for L in self.layers:
                L["wqkv"].mul_(L["ln1"][None, :])
                L["wgu"].mul_(L["ln2"][None, :])
            self.norms_folded = True
        return self

    def can_pack_linear(self) -> bool:
        c = self.cfg
        qkv, o = (c.hq + 2 * c.hkv) * c.head_dim, c.hq * c.head_dim
        return (self.norms_folded and self.embed.dtype == torch.bfloat16 and c.hidden % 32 == 0 and o % 32 == 0 and qkv % 16 == 0
                and c.intermediate % 32 == 0 and (c.intermediate % 24 == 0 or c.intermediate % 16 == 0))

    def pack_linear(self) -> "Weights":
        """A second copy of every layer's four weights in the order ``ops.linear_rows`` streams them (``wqkv_p``,
        ``wo_p``, ``wgu_p``, ``wdown_p``), made once; needs the input norms folded in (``wgu`` carries ln2).  The
        row-major weights stay for prefill."""
        if not self.linear_packed:
            if not self.can_pack_linear():
                raise TahDuoError("pack_linear: needs folded input norms, bf16 and sizes in whole MFMA steps")
            for L in self.layers:
                L["wqkv_p"] = ops.linear_pack_weight(L["wqkv"])
                L["wo_p"] = ops.linear_pack_weight(L["wo"])
                L["wgu_p"] = ops.linear_pack_weight(L["wgu"], gate_up=True)
                L["wdown_p"] = ops.linear_pack_weight(L["wdown"])
            # the output head with the final norm's weight inside (a copy: the head may be the embedding itself)
            self.lm_head_p = ops.linear_pack_weight(self.lm_head * self.norm[None, :]) if self.cfg.vocab % 16 == 0 else None
            # the decider's first layer behind the final norm, the same way
            self.dec_w1_p = (ops.linear_pack_weight(self.dec_w1 * self.norm[None, :])
                             if self.dec_w1 is not None and self.dec_w1.shape[0] % 16 == 0 else None)
            self.linear_packed = True
        return self

    @staticmethod
    def random_init(cfg: EngineConfig, device, seed: int = 0, dtype=torch.bfloat16) -> "Weights":
        gdev = torch.device(device)
        g = torch.Generator(device=gdev).manual_seed(seed)  # drawn where the weights live (1.7 G values at full size)
        w = Weights(cfg)

        def lin(o, i, std=None):
            std = std if std is not None else 1.0 / math.sqrt(i)
            out = torch.empty(o, i, dtype=dtype, device=gdev)
            rows = max(1, (1 << 26) // i)  # in pieces: the float32 draws stay small
            for r in range(0, o, rows):
                n = min(rows, o - r)
                out[r:r + n] = (torch.randn(n, i, generator=g, device=gdev) * std).to(dtype)
            return out

        H, D, I = cfg.hidden, cfg.head_dim, cfg.intermediate
        w.embed = lin(cfg.vocab, H, std=0.02)
        w.lm_head = w.embed
        ones = lambda n: (1.0 + 0.05 * torch.randn(n, generator=g, device=gdev)).to(dtype)
        w.norm = ones(H)
        for _ in range(cfg.layers):
            w.layers.append(dict(ln1=ones(H), wqkv=lin((cfg.hq + 2 * cfg.hkv) * D, H), qn=ones(D), kn=ones(D),
                                 wo=lin(H, cfg.hq * D), ln2=ones(H), wgu=lin(2 * I, H), wdown=lin(H, I)))
        w.dec_w1, w.dec_b1 = lin(cfg.decider_hidden, H), torch.zeros(cfg.decider_hidden, dtype=dtype, device=gdev)
        w.dec_w2, w.dec_b2 = lin(1, cfg.decider_hidden), torch.zeros(1, dtype=dtype, device=gdev)
        return w

    @staticmethod
    def from_hf(model, cfg: EngineConfig, device, dtype=torch.bfloat16) -> "Weights":
        """Copies the tensors of a Hugging Face ``Qwen3ForCausalLM`` (q/k/v and gate/up fused row-wise)."""
        w = Weights(cfg)
        t = lambda x: x.detach().to(device=device, dtype=dtype).contiguous()
        base = model.model
        w.embed, w.norm = t(base.embed_tokens.weight), t(base.norm.weight)
        w.lm_head = w.embed if model.lm_head.weight is base.embed_tokens.weight else t(model.lm_head.weight)
        for lyr in base.layers:
            a, m = lyr.self_attn, lyr.mlp
            w.layers.append(dict(
                ln1=t(lyr.input_layernorm.weight),
                wqkv=t(torch.cat([a.q_proj.weight, a.k_proj.weight, a.v_proj.weight], 0)),
                qn=t(a.q_norm.weight), kn=t(a.k_norm.weight), wo=t(a.o_proj.weight),
                ln2=t(lyr.post_attention_layernorm.weight),
                wgu=t(torch.cat([m.gate_proj.weight, m.up_proj.weight], 0)), wdown=t(m.down_proj.weight)))
        return w


def rope_tables(max_len: int, head_dim: int, theta: float, device, dtype=torch.bfloat16) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos / sin rows as ``Qwen3RotaryEmbedding`` produces them (float32 angles, cast to the model dtype)."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    ang = torch.arange(max_len, dtype=torch.float32)[:, None] * inv[None]
    emb = torch.cat([ang, ang], -1)
    return emb.cos().to(dtype).to(device), emb.sin().to(dtype).to(device)


class TaHDecodeEngine:
    def __init__(self, weights: Weights, batch: int, max_len: int, *, max_hard: Optional[int] = None, device="cuda",
                 fold_norms: bool = True, packed_linear: bool = True, decider=None):
        """``fold_norms``: multiply the layers' input-norm weights into the projections behind them (in place in
        ``weights``, once) so that the two RMSNorms of a layer cost no launch; needs hidden % 8 == 0 and bf16.
        ``packed_linear``: run the linear layers of a decode step on ``ops.linear_rows`` (a second, re-ordered copy
        of the layers' weights is made once); needs ``fold_norms``, at most 32 rows and sizes in whole MFMA steps,
        otherwise the step keeps torch GEMMs.  ``decider``: a ``tah_amd.decider.MLPIterDecider`` (the reference's learned
        decider, iter_decider.py:193-301) to decide with instead of the two-layer MLP in ``weights``: it sees each token's
        first-iteration logits and the hidden states of its configured layers, counted as Hugging Face's
        ``output_hidden_states`` counts them (0: the embeddings, i: after layer i, the last one after the final norm;
        tah_model.py:434-441, 615-642)."""
        cfg = weights.cfg
        if cfg.head_dim != 128:
            raise TahDuoError("the kernels are built for head_dim 128")
        if fold_norms and cfg.hidden % 8 == 0 and weights.embed.dtype == torch.bfloat16:
            weights.fold_norms()
        self.packed_linear = bool(packed_linear and batch <= ops.LINEAR_MAX_ROWS and weights.can_pack_linear())
        if self.packed_linear:
            weights.pack_linear()
        self.w, self.cfg, self.B, self.max_len = weights, cfg, batch, max_len
        self.device = torch.device(device)
        self.max_hard = max_hard if max_hard is not None else max_len
        self.cos, self.sin = rope_tables(max_len, cfg.head_dim, cfg.rope_theta, self.device)
        self.slabs0 = [KvSlabs(batch, max_len, cfg.hkv, cfg.head_dim, with_pos=False, device=self.device) for _ in range(cfg.layers)]
        self.slabs1 = [KvSlabs(batch, self.max_hard, cfg.hkv, cfg.head_dim, with_pos=True, device=self.device) for _ in range(cfg.layers)]
        dev = self.device
        self.rows = torch.arange(batch, dtype=torch.int32, device=dev)
        self.cu_rows = torch.arange(batch + 1, dtype=torch.int32, device=dev)
        self.minus1 = torch.full((batch,), -1, dtype=torch.int32, device=dev)
        self.zeros_i = torch.zeros(batch, dtype=torch.int32, device=dev)
        # generation state (all on the device)
        self.fused_greedy = True  # arg-max + bookkeeping of a greedy step in one launch (tah_greedy_step)
        self.fused_sampling = True  # draws without a top-k filter in one launch (tah_sample_rows) instead of a sort in torch
        self.use_fused_glue = True  # (tests switch it off to compare with the torch glue)
        self.tok = torch.zeros(batch, dtype=torch.long, device=dev)       # token fed to the next step
        self.pos = torch.zeros(batch, dtype=torch.int32, device=dev)      # its position
        self.finished = torch.zeros(batch, dtype=torch.bool, device=dev)
        self.n_hard = torch.zeros((), dtype=torch.long, device=dev)       # tokens that took a second iteration
        self.n_steps = torch.zeros((), dtype=torch.long, device=dev)      # tokens decoded (active rows x steps)
        self.step_idx = torch.zeros(1, dtype=torch.long, device=dev)
        self.out_tokens = torch.zeros(batch, max_len, dtype=torch.long, device=dev)  # generated tokens, column = step
        self.out_len = torch.zeros(batch, dtype=torch.int32, device=dev)             # tokens of each row before its end
        self.scale = float(cfg.head_dim) ** -0.5
        self.host_positions = 0  # upper bound on any sequence's length, kept on the host for capacity checks
        self.host_hard_rows = 0
        self._graph = None
        self.static_scratch = self.device.type == "cuda"
        self.measure_without_attention = False
        # depth-1 rows every sequence has cached (what each slabs1[l].len holds), kept once for the fused step kernel
        self.hard_len = torch.zeros(batch, dtype=torch.int32, device=dev)
        # q/k preparation, append and attention of a layer in one launch where the library takes the sizes
        self.fused_step = bool(self.packed_linear and self.device.type == "cuda"
                               and decode_step_supported(batch, cfg.hq, cfg.hkv, max_len))
        if self.packed_linear:  # rows operands handed from kernel to kernel (32 rows each; rows past the batch stay zero)
            z = lambda n: torch.zeros(32 * n, dtype=torch.bfloat16, device=dev)
            self.xp, self.op, self.actp = z(cfg.hidden), z(cfg.hq * cfg.head_dim), z(cfg.intermediate)
        # the step's element-wise glue in two launches (tah_step_begin, tah_decider_tail) and the decider's first layer
        # on the linear-layer kernel, instead of some twenty torch launches; needs the packed rows
        self.fused_glue = bool(self.packed_linear and weights.lm_head_p is not None and
                               (decider is not None or (weights.dec_w1_p is not None and cfg.decider_hidden % 8 == 0)))
        if self.fused_glue:
            i32 = lambda: torch.zeros(batch, dtype=torch.int32, device=dev)
            self.x0 = torch.zeros(batch, cfg.hidden, dtype=torch.bfloat16, device=dev)
            self.x1 = torch.zeros_like(self.x0)
            self.cos_rows = torch.zeros(batch, cfg.head_dim, dtype=torch.bfloat16, device=dev)
            self.sin_rows = torch.zeros_like(self.cos_rows)
            self.slot0, self.qpos0, self.slot1, self.qpos1, self.hard_i = i32(), i32(), i32(), i32(), i32()
            self.act = torch.zeros(batch, dtype=torch.bool, device=dev)
            self.hard = torch.zeros(batch, dtype=torch.bool, device=dev)
        # Rows at different latent iterations in one batch (generate(..., continuous=True)): a row whose token takes no
        # second iteration goes on to its next token while others run theirs.  Needs the fused attention launch (it
        # appends per row to the depth-0 or depth-1 slabs) and the fused glue.
        self.can_run_continuous = bool(self.fused_glue and self.fused_step)
        self.phase = torch.zeros(batch, dtype=torch.int32, device=dev)   # 1: the row's next pass is a second iteration
        if self.can_run_continuous:
            self.q_depth_rows, self.append_at = i32(), i32()
            self.eligible = torch.zeros(batch, dtype=torch.bool, device=dev)
            self.logits2 = [torch.zeros(batch, cfg.vocab, dtype=torch.bfloat16, device=dev) for _ in range(2)]
        self._tick_graphs = None
        self.decider = decider
        if decider is not None:
            if decider.hidden_states_size != cfg.hidden:
                raise TahDuoError("the decider's hidden_states_size differs from the model's hidden size")
            self.hs_pick = list(decider.hidden_states_layer_nums) or [cfg.layers]
            if min(self.hs_pick) < 0 or max(self.hs_pick) > cfg.layers:
                raise TahDuoError("the decider's hidden_states_layer_nums do not fit the model's layers")
            # what the last single-token pass left: [B, picked layers, H], and the decision logits of the last decision
            self.hs_buf = torch.zeros(batch, len(self.hs_pick), cfg.hidden, dtype=weights.embed.dtype, device=dev)
            self.decision_logits = None

    def _keep_hidden(self, index: int, x: torch.Tensor, into: Optional[list] = None):
        """Called with the hidden state after ``index`` layers (before the final norm): keeps it if the decider wants it."""
        if self.decider is None or index not in self.hs_pick:
            return
        h = self._rms(x, self.w.norm) if index == self.cfg.layers else x
        for j, want in enumerate(self.hs_pick):
            if want == index:
                if into is None:
                    self.hs_buf[:, j].copy_(h)
                else:
                    into[j] = h

    def _decide_rows(self, logits: torch.Tensor, hidden_states: torch.Tensor):
        """The learned decider after a token's first iteration (iter_depth 1 of at most 2: tah_model.py:625-642)."""
        mask, z = self.decider.decide_selected(logits, 1, hidden_states.reshape(hidden_states.shape[0], -1))
        self.decision_logits = z
        return mask

    # ── model pieces ─────────────────────────────────────────────────────
    def _rms(self, x, w):
        return F.rms_norm(x, (x.shape[-1],), w, self.cfg.rms_eps)

    def _mlp(self, x, L):
        if self.w.norms_folded:  # the norm's weight sits in wgu, its per-row factor is applied with the gate
            h = ops.silu_mul(x @ L["wgu"].t(), norm_input=x, norm_eps=self.cfg.rms_eps)
        else:
            h = ops.silu_mul(self._rms(x, L["ln2"]) @ L["wgu"].t())
        return x.addmm_(h, L["wdown"].t())

    def _prefill_qkv(self, x, L, cos, sin):
        """Prepared q, k and v of packed prompt rows (input norm, projections, q/k norm, rotary embedding)."""
        c = self.cfg
        if self.w.norms_folded:
            q, k, v = self._split_qkv(x @ L["wqkv"].t())
            return qk_norm_rope(q, k, L["qn"], L["kn"], cos, sin, c.rms_eps, v=v, norm_input=x, norm_eps=c.rms_eps)
        q, k, v = self._split_qkv(self._rms(x, L["ln1"]) @ L["wqkv"].t())
        qo, ko = qk_norm_rope(q, k, L["qn"], L["kn"], cos, sin, c.rms_eps)
        return qo, ko, v

    def _split_qkv(self, qkv):
        c = self.cfg
        n = qkv.shape[0]
        qkv = qkv.view(n, c.hq + 2 * c.hkv, c.head_dim)
        return qkv[:, :c.hq], qkv[:, c.hq:c.hq + c.hkv], qkv[:, c.hq + c.hkv:]

    def decide(self, hidden: torch.Tensor) -> torch.Tensor:
        """Continue probability of the two-layer decider MLP on the last hidden state, float32 [rows]."""
        w = self.w
        h = F.relu(hidden @ w.dec_w1.t() + w.dec_b1)
        return torch.sigmoid((h @ w.dec_w2.t() + w.dec_b2).float()).view(-1)

    # ── one token per sequence through all layers at one depth ───────────
    def _rope_rows(self, pos):
        at = pos.long().clamp(0, self.max_len - 1)  # a position past the tables (a caller replaying beyond the
        return self.cos[at], self.sin[at]           # capacity) must not read outside them

    def _pass_single(self, x, pos, depth: int, slot_of, q_pos, q_depth, rope=None):
        """x [B, H]; appends this token's K/V to the depth's slabs (rows with slot_of < 0 are not cached) and
        attends with q_pos / q_depth per row (q_pos < 0: the row sees nothing and is dropped by the caller).  Returns
        the final-normed hidden state (with packed linear layers: the hidden state before the final norm, see
        ``_head``)."""
        c = self.cfg
        cos, sin = rope if rope is not None else self._rope_rows(pos)
        if self.packed_linear:
            return self._pass_single_packed(x, pos, depth, slot_of, q_pos, q_depth, cos, sin)
        folded = self.w.norms_folded
        self._keep_hidden(0, x)
        for l, L in enumerate(self.w.layers):
            qkv = (x if folded else self._rms(x, L["ln1"])) @ L["wqkv"].t()
            q, k, v = self._split_qkv(qkv)
            cache = self.slabs0[l] if depth == 0 else self.slabs1[l]
            if self.measure_without_attention:  # timing aid: the step minus its q/k preparation and decode kernels
                o = q.contiguous()
            else:
                qo, _ = qk_norm_rope(q, k, L["qn"], L["kn"], cos, sin, c.rms_eps, v=v, cache=cache, cu_new=self.cu_rows,
                                     slot_of=slot_of, pos_new=pos if depth == 1 else None, one_row_per_seq=True,
                                     norm_input=x if folded else None, norm_eps=c.rms_eps)
                o = _decode(qo, self.rows, q_pos, self.slabs0[l], self.slabs1[l], scale=self.scale, q_depth=q_depth,
                            static_scratch=self.static_scratch)
            x = x.addmm_(o.view(x.shape[0], c.hq * c.head_dim), L["wo"].t())  # residual add inside the GEMM, in place
            x = self._mlp(x, L)
            self._keep_hidden(l + 1, x)
        return self._rms(x, self.w.norm)

    def _pass_single_packed(self, x, pos, depth: int, slot_of, q_pos, q_depth, cos, sin, rows_packed: bool = False):
        """The same pass with the four linear layers of a layer on ``ops.linear_rows``: seven launches per layer.  The
        hidden state lives twice, row-major in ``x`` (updated in place; read by the q/k preparation for the norm
        factor) and as rows operand in ``self.xp``; attention output and MLP activation exist as rows operands only."""
        c = self.cfg
        B, H, I = x.shape[0], c.hidden, c.intermediate
        n_qkv, n_o = (c.hq + 2 * c.hkv) * c.head_dim, c.hq * c.head_dim
        x = x.contiguous()
        xp = self.xp if rows_packed else ops.linear_pack_rows(x, out=self.xp)  # rows_packed: self.xp already holds x
        self._keep_hidden(0, x)
        for l, L in enumerate(self.w.layers):
            q, k, v = self._split_qkv(ops.linear_rows(L["wqkv_p"], xp, B, n_qkv, H))
            cache = self.slabs1[l] if depth == 1 else self.slabs0[l]
            if self.measure_without_attention:  # timing aid: the step minus its q/k preparation and decode kernels
                ops.linear_pack_rows(q.reshape(B, n_o), out=self.op)
            elif depth is None:  # every row at its own iteration (q_depth): it appends to that depth's slabs
                _decode_step(q, k, v, L["qn"], L["kn"], cos, sin, c.rms_eps, cache=self.slabs1[l], cu_new=self.cu_rows,
                             append_at=self.append_at, append_depth=q_depth, q_slot=self.rows, q_pos=q_pos,
                             c1=self.slabs0[l], c2=self.slabs1[l], scale=self.scale, slot_of=slot_of, pos_new=pos,
                             norm_input=x, norm_eps=c.rms_eps, q_depth=q_depth, out_packed=self.op)
            elif self.fused_step:
                _decode_step(q, k, v, L["qn"], L["kn"], cos, sin, c.rms_eps, cache=cache, cu_new=self.cu_rows,
                             append_at=pos if depth == 0 else self.hard_len, q_slot=self.rows, q_pos=q_pos,
                             c1=self.slabs0[l], c2=self.slabs1[l], scale=self.scale, slot_of=slot_of,
                             pos_new=pos if depth == 1 else None, norm_input=x, norm_eps=c.rms_eps, q_depth=q_depth,
                             out_packed=self.op)
            else:
                qo, _ = qk_norm_rope(q, k, L["qn"], L["kn"], cos, sin, c.rms_eps, v=v, cache=cache, cu_new=self.cu_rows,
                                     slot_of=slot_of, pos_new=pos if depth == 1 else None, one_row_per_seq=True,
                                     norm_input=x, norm_eps=c.rms_eps)
                _decode(qo, self.rows, q_pos, self.slabs0[l], self.slabs1[l], scale=self.scale, q_depth=q_depth,
                        static_scratch=self.static_scratch, out_packed=self.op)
            ops.linear_rows(L["wo_p"], self.op, B, H, n_o, residual=x, out=x, out_packed=xp)
            ops.linear_rows(L["wgu_p"], xp, B, I, H, gate_up=True, out_packed=self.actp, want_out=False, norm_eps=c.rms_eps)
            ops.linear_rows(L["wdown_p"], self.actp, B, H, I, residual=x, out=x, out_packed=xp)
            self._keep_hidden(l + 1, x)
        return x  # before the final norm; self.xp holds the same rows as operand

    def _head(self, h):
        """Logits [B, V] of what a pass returned: the final-normed rows through the head, or, with packed linear
        layers, the rows operand the last layer left in ``self.xp`` through the head that carries the final norm's
        weight, the norm's factor applied to the products."""
        c = self.cfg
        if not self.packed_linear:
            return h @ self.w.lm_head.t()
        if self.w.lm_head_p is None:
            return self._rms(h, self.w.norm) @ self.w.lm_head.t()
        return ops.linear_rows(self.w.lm_head_p, self.xp, h.shape[0], c.vocab, c.hidden, norm_eps=c.rms_eps)

    def step_logits(self, tok: torch.Tensor, force_hard: Optional[torch.Tensor] = None, active: Optional[torch.Tensor] = None):
        """The iteration loop of tah_model.py:580-706 for one new token per sequence, on ``self.pos``.

        Returns (final logits float32 [B, V], hard bool [B]).  ``force_hard`` replaces the decider's decision
        (tests drive both implementations with the same decisions).  Rows that are not ``active`` are neither
        cached nor attended; their logits are meaningless."""
        l0, l1, hard = self._step_parts(tok, force_hard, active)
        # running sum of the iterations' logits, rounded to the model dtype as the reference's buffers are
        # (tah_model.py:543, 628)
        return torch.where(hard[:, None], (l0 + l1).float(), l0.float()), hard

    def _step_parts(self, tok: torch.Tensor, force_hard: Optional[torch.Tensor] = None, active: Optional[torch.Tensor] = None):
        """Both latent iterations of one step: logits of the first and of the second iteration (model dtype [B, V];
        the second are meaningless for rows that are not hard) and hard bool [B]."""
        B = self.B
        pos = self.pos
        act = active if active is not None else torch.ones(B, dtype=torch.bool, device=self.device)
        slot0 = torch.where(act, self.rows, self.minus1)
        qpos0 = torch.where(act, pos, self.minus1)
        rope = self._rope_rows(pos)  # both latent iterations of a token use its position
        h0 = self._pass_single(self.w.embed[tok], pos, 0, slot0, qpos0, self.zeros_i, rope)
        l0 = self._head(h0)
        if self.packed_linear:
            h0 = self._rms(h0, self.w.norm)
        if force_hard is not None:
            hard = force_hard
            if self.decider is not None:
                self._decide_rows(l0, self.hs_buf)  # (kept for inspection: decision_logits)
        elif self.decider is not None:
            hard = self._decide_rows(l0, self.hs_buf)
        else:
            hard = self.decide(h0) > self.w.threshold
        hard = hard & act
        # next-iteration input of the hard rows (tah_model.py:693-697); the other rows keep zeros
        x1 = ops.topk_mix(l0, self.w.embed, self.cfg.topk, row_enable=hard)
        slot1 = torch.where(hard, self.rows, self.minus1)
        qpos1 = torch.where(hard, pos, self.minus1)
        hard_i = hard.to(torch.int32)
        h1 = self._pass_single(x1, pos, 1, slot1, qpos1, hard_i, rope)
        self.hard_len += hard_i  # after all layers appended at the old count
        return l0, self._head(h1), hard

    def _step_parts_device(self):
        """``_step_parts(self.tok, active=~self.finished)`` with the element-wise glue in two launches and the decider's
        first layer on the linear-layer kernel (the final norm folded into it, as into the output head): the decider sees
        the same numbers up to bf16 rounding order."""
        c, w, B = self.cfg, self.w, self.B
        ops.step_begin(self.tok, self.pos, self.finished, w.embed, self.cos, self.sin, x=self.x0, x_packed=self.xp,
                       cos_rows=self.cos_rows, sin_rows=self.sin_rows, slot=self.slot0, q_pos=self.qpos0, active=self.act)
        self._pass_single_packed(self.x0, self.pos, 0, self.slot0, self.qpos0, self.zeros_i, self.cos_rows, self.sin_rows,
                                 rows_packed=True)
        l0 = self._head(self.x0)
        if self.decider is not None:
            torch.logical_and(self._decide_rows(l0, self.hs_buf), self.act, out=self.hard)
            self.hard_i.copy_(self.hard)
            torch.where(self.hard, self.rows, self.minus1, out=self.slot1)
            torch.where(self.hard, self.pos, self.minus1, out=self.qpos1)
        else:
            hr = ops.linear_rows(w.dec_w1_p, self.xp, B, c.decider_hidden, c.hidden, norm_eps=c.rms_eps, bias=w.dec_b1, relu=True)
            ops.decider_tail(hr, w.dec_w2.reshape(-1), w.dec_b2, w.threshold, hard=self.hard, active=self.act, pos=self.pos,
                             hard_i32=self.hard_i, slot=self.slot1, q_pos=self.qpos1)
        ops.topk_mix(l0, w.embed, c.topk, row_enable=self.hard, out=self.x1, out_packed=self.xp, zero_disabled=True)
        h1 = self._pass_single_packed(self.x1, self.pos, 1, self.slot1, self.qpos1, self.hard_i, self.cos_rows, self.sin_rows,
                                      rows_packed=True)
        self.hard_len += self.hard_i  # after all layers appended at the old count
        return l0, self._head(h1), self.hard

    def _parts(self):
        """Both iterations of a step on the engine's own state: (logits0, logits1, hard, active)."""
        if self.fused_glue and self.use_fused_glue:
            return self._step_parts_device() + (self.act,)
        act = ~self.finished
        return self._step_parts(self.tok, active=act) + (act,)

    # ── prefill: packed prompts, both depths, through the varlen kernels ──
    @torch.no_grad()
    def prefill(self, ids: torch.Tensor, cu: torch.Tensor, *, force_hard: Optional[torch.Tensor] = None,
                calibrate: Optional[float] = None):
        """ids int64 [N] (the prompts one after another), cu int32 [B+1].  Fills both caches and returns
        (logits float32 [B, V] of each prompt's last token, hard bool [N]).  ``calibrate=p`` first sets the
        decider threshold to the (1-p) quantile of its outputs on these prompts."""
        c, w, dev = self.cfg, self.w, self.device
        B = self.B
        if cu.numel() != B + 1:
            raise TahDuoError("cu must have batch + 1 entries")
        cu_h = cu.cpu()
        lens = (cu_h[1:] - cu_h[:-1]).tolist()
        N = int(cu_h[-1])
        if max(lens) > self.max_len:
            raise TahDuoError("prompt longer than the cache capacity")
        # a new batch: whatever an earlier generation left in the slabs is forgotten
        for sl in self.slabs0 + self.slabs1:
            sl.len.zero_()
            sl.overflow.zero_()
        self.n_hard.zero_()
        self.n_steps.zero_()
        self.host_hard_rows = 0
        self._graph = None  # (its warm-up step belongs to the old batch's state)
        self._tick_graphs = None
        self.phase.zero_()
        seq = torch.repeat_interleave(torch.arange(B, device=dev), torch.tensor(lens, device=dev))
        pos = (torch.arange(N, device=dev) - cu.long()[seq]).to(torch.int32)
        cos, sin = self.cos[pos.long()], self.sin[pos.long()]
        zc = torch.zeros(B + 1, dtype=torch.int32, device=dev)
        zi = torch.zeros(0, dtype=torch.int32, device=dev)
        x = w.embed[ids]
        kv_tok = []
        hs_sel = [None] * len(self.hs_pick) if self.decider is not None else None
        self._keep_hidden(0, x, hs_sel)
        # launch order of the prompts' tiles, heaviest first across prompts: one table serves all layers of a depth
        sched0 = ops.duo_schedule(cu, cu, zc, zc, zi, c.hq, c.hkv, N, N, 0)
        for l, L in enumerate(w.layers):
            qo, ko, v = self._prefill_qkv(x, L, cos, sin)
            o1, _, _, _ = ops.duo_fwd_varlen(qo, ko, v, cu, cu, qo[:0], ko[:0], v[:0], zi, zi, zc, zc, self.scale,
                                             schedule=sched0)
            self.slabs0[l].append(ko, v, cu)
            kv_tok.append((ko, v))
            x = x + o1.view(N, -1) @ L["wo"].t()
            x = self._mlp(x, L)
            self._keep_hidden(l + 1, x, hs_sel)
        h0 = self._rms(x, w.norm)
        if self.decider is not None:
            # the decider wants every prompt token's logits: a thousand rows of the vocabulary at a time
            zs = []
            for a in range(0, N, 1024):
                b = min(a + 1024, N)
                self._decide_rows(h0[a:b] @ w.lm_head.t(), torch.stack([h[a:b] for h in hs_sel], dim=1))
                zs.append(self.decision_logits)
            z = self.decision_logits = torch.cat(zs)
            prob = torch.sigmoid(z)  # in the logits' dtype, as the decider compares it (iter_decider.py:299)
            if calibrate is not None:
                with torch.no_grad():
                    self.decider.threshold.fill_(float(torch.quantile(prob.float(), 1.0 - calibrate)))
            hard = (prob > self.decider.threshold.to(z.dtype)) if force_hard is None else force_hard
        else:
            prob = self.decide(h0)
            if calibrate is not None:
                w.threshold = float(torch.quantile(prob, 1.0 - calibrate))
            hard = (prob > w.threshold) if force_hard is None else force_hard
        last = (cu[1:] - 1).long()
        logits_last = (h0[last] @ w.lm_head.t())  # model dtype, like the reference's logits buffers
        rows2 = torch.nonzero(hard).flatten()
        n2 = rows2.numel()
        if n2:
            counts = torch.zeros(B, dtype=torch.long, device=dev).index_add_(0, seq[rows2], torch.ones_like(rows2))
            if int(counts.max()) > self.max_hard:
                raise TahDuoError("more hard tokens in a prompt than the depth-1 cache holds")
            cu2 = torch.cat([torch.zeros(1, dtype=torch.long, device=dev), counts.cumsum(0)]).to(torch.int32)
            l0h = h0[rows2] @ w.lm_head.t()
            x2 = ops.topk_mix(l0h, w.embed, c.topk)
            pos2 = pos[rows2].contiguous()
            cos2, sin2 = self.cos[pos2.long()], self.sin[pos2.long()]
            sched1 = ops.duo_schedule(zc, cu, cu2, cu2, pos2, c.hq, c.hkv, 0, N, n2)
            for l, L in enumerate(w.layers):
                qo, ko, v = self._prefill_qkv(x2, L, cos2, sin2)
                k1, v1 = kv_tok[l]
                _, _, o2, _ = ops.duo_fwd_varlen(qo[:0], k1, v1, zc, cu, qo, ko, v, pos2, pos2, cu2, cu2, self.scale,
                                                 schedule=sched1)
                self.slabs1[l].append(ko, v, cu2, pos_new=pos2)
                x2 = x2 + o2.view(n2, -1) @ L["wo"].t()
                x2 = self._mlp(x2, L)
            l1h = self._rms(x2, w.norm) @ w.lm_head.t()
            both = l0h + l1h
            # a prompt whose last token is hard: its final logits are the sum of both iterations'
            is_last = torch.isin(rows2, last)
            if bool(is_last.any()):
                which = seq[rows2[is_last]]
                logits_last[which] = both[is_last]
            self.host_hard_rows = int(counts.max())
        self.pos.copy_(torch.tensor(lens, dtype=torch.int32))
        self.hard_len.copy_(self.slabs1[0].len)
        self.host_positions = max(lens)
        self.finished.zero_()
        return logits_last.float(), hard

    # ── sampling / generation ────────────────────────────────────────────
    @staticmethod
    def sample(logits: torch.Tensor, temperature: float = 0.0, *, top_p: float = 1.0, top_k: int = 0, min_p: float = 0.0) -> torch.Tensor:
        """One token per row, batched on the device: ``sample_next_token`` of the reference
        (tah/model/utils.py:84-125) -- temperature, softmax, then min_p / top_k / top_p filters with
        renormalisation, then one draw per row -- with ``temperature <= 0`` meaning ``do_sample=False`` (arg-max).
        The draw is the exponential-race form of a multinomial draw (arg-max of p / e, e ~ Exp(1)), which can be
        captured in a graph."""
        if temperature <= 0.0:
            return torch.argmax(logits, dim=-1)
        probs = TaHDecodeEngine.filtered_probs(logits, temperature, top_p=top_p, top_k=top_k, min_p=min_p)
        return torch.argmax(probs / torch.empty_like(probs).exponential_(), dim=-1)

    @staticmethod
    def filtered_probs(logits: torch.Tensor, temperature: float, *, top_p: float = 1.0, top_k: int = 0, min_p: float = 0.0) -> torch.Tensor:
        """The distribution ``sample`` draws from: [rows, V], zero outside the filters."""
        probs = F.softmax(logits / temperature if temperature != 1.0 else logits, dim=-1)
        if min_p > 0.0:
            probs = torch.where(probs >= min_p * probs.max(dim=-1, keepdim=True).values, probs, torch.zeros_like(probs))
            probs = probs / probs.sum(dim=-1, keepdim=True)
        if top_k > 0:
            kth = torch.topk(probs, min(top_k, probs.size(-1)), dim=-1).values[..., -1:]
            probs = torch.where(probs < kth, torch.zeros_like(probs), probs)
            probs = probs / probs.sum(dim=-1, keepdim=True)
        if top_p < 1.0:
            sp, si = torch.sort(probs, descending=True, dim=-1)
            remove = torch.cumsum(sp, dim=-1) > top_p
            remove = torch.cat([torch.zeros_like(remove[..., :1]), remove[..., :-1]], dim=-1)  # keep the one that crosses
            probs = torch.where(torch.zeros_like(remove).scatter_(-1, si, remove), torch.zeros_like(probs), probs)
            probs = probs / probs.sum(dim=-1, keepdim=True)
        return probs

    # With a top-k filter (0 < top_k <= 256) nothing outside the k largest logits can be drawn, and every filter compares
    # probabilities with each other, never with the softmax's denominator: the whole of ``sample`` can run on the
    # [rows, k] values that one ``tah_topk_mix`` launch returns (largest first, with their vocabulary indices) instead
    # of on [rows, V] -- no sort over the vocabulary, about a millisecond less per step at 32 x 151 936.  One
    # difference: logits equal to the k-th largest beyond the k-th place stay out (the lower indices are taken),
    # where ``torch.where(probs < kth, 0, probs)`` (utils.py:113) keeps them all.
    TOPK_SAMPLING_MAX = 256

    @staticmethod
    def topk_filtered_probs(vals: torch.Tensor, temperature: float, *, top_p: float = 1.0, min_p: float = 0.0) -> torch.Tensor:
        """``filtered_probs`` on the k largest logits of every row, ``vals`` [rows, k] sorted largest first."""
        x = vals.float()
        probs = F.softmax(x / temperature if temperature != 1.0 else x, dim=-1)
        if min_p > 0.0:
            probs = torch.where(probs >= min_p * probs[..., :1], probs, torch.zeros_like(probs))
            probs = probs / probs.sum(dim=-1, keepdim=True)
        if top_p < 1.0:
            remove = torch.cumsum(probs, dim=-1) > top_p
            remove = torch.cat([torch.zeros_like(remove[..., :1]), remove[..., :-1]], dim=-1)  # keep the one that crosses
            probs = torch.where(remove, torch.zeros_like(probs), probs)
            probs = probs / probs.sum(dim=-1, keepdim=True)
        return probs

    @staticmethod
    def sample_topk(logits: torch.Tensor, temperature: float, *, top_p: float = 1.0, top_k: int, min_p: float = 0.0) -> torch.Tensor:
        """``sample`` for bf16 logits [rows, V] and 0 < top_k <= TOPK_SAMPLING_MAX."""
        vals, idx = ops.topk(logits, top_k)
        probs = TaHDecodeEngine.topk_filtered_probs(vals, temperature, top_p=top_p, min_p=min_p)
        j = torch.argmax(probs / torch.empty_like(probs).exponential_(), dim=-1, keepdim=True)
        return torch.gather(idx, 1, j).squeeze(1).to(torch.int64)

    # Without a top-k filter the draw is one ``tah_sample_rows`` launch on the bf16 logits (no sort over the vocabulary);
    # with one of at most 256 places it runs on the k largest logits; anything else takes the torch formulation.
    SAMPLE_ROWS_MAX_VOCAB = 155648

    def _draw(self, logits: torch.Tensor, temperature: float, prev: Optional[torch.Tensor] = None,
              add_prev: Optional[torch.Tensor] = None, **filters) -> torch.Tensor:
        """One token per row from final logits in bf16.  ``prev`` / ``add_prev`` (int32 [rows]): rows whose entry is not 0
        draw from ``prev + logits``, summed in bf16 as the step-wise loop forms the final logits of a hard token."""
        k = int(filters.get("top_k", 0))
        fits = logits.dtype == torch.bfloat16 and logits.size(-1) <= self.SAMPLE_ROWS_MAX_VOCAB
        if k == 0 and fits and self.fused_sampling:
            u = torch.rand(logits.size(0), dtype=torch.float32, device=logits.device)
            return ops.sample_rows(logits, u, temperature, top_p=float(filters.get("top_p", 1.0)), min_p=float(filters.get("min_p", 0.0)),
                                   logits_prev=prev, add_prev=add_prev)
        final = logits if prev is None else torch.where((add_prev != 0)[:, None], prev + logits, logits)
        if 0 < k <= self.TOPK_SAMPLING_MAX and fits:
            return self.sample_topk(final, temperature, **filters)
        return self.sample(final.float(), temperature, **filters)

    def _step_inplace(self, temperature: float, eos: int, **filters):
        """One generated token for every unfinished row; every state change is an in-place device update."""
        l0, l1, hard, act = self._parts()
        if temperature <= 0.0 and self.fused_greedy and self.w.embed.dtype == torch.bfloat16 and self.cfg.vocab % 8 == 0:
            # arg-max of the final logits and the bookkeeping below in one launch; the final logits are not formed
            ops.greedy_step(l0, l1, hard, eos, self.tok, self.finished, self.pos, self.out_tokens, self.step_idx, self.out_len,
                            self.n_hard, self.n_steps)
            self.step_idx += 1
            return
        if temperature > 0.0:  # final logits as step_logits forms them: l0, plus l1 for hard tokens (the sum in the logits' dtype)
            nxt = self._draw(l0, temperature, prev=l1, add_prev=hard.to(torch.int32), **filters)
        else:
            nxt = self.sample(torch.where(hard[:, None], l0 + l1, l0).float(), 0.0)
        nxt = torch.where(act, nxt, torch.zeros_like(nxt))
        if eos >= 0:
            self.finished |= nxt == eos
        # a row's output ends before its end-of-sequence token (utils.py:241-245); finished rows write zeros
        keep = ~self.finished
        self.out_tokens.scatter_(1, self.step_idx.expand(self.B, 1), torch.where(keep, nxt, torch.zeros_like(nxt))[:, None])
        self.out_len += keep.to(torch.int32)
        self.n_hard += hard.sum()
        self.n_steps += act.sum()
        self.pos += act.to(torch.int32)
        self.step_idx += 1
        self.tok.copy_(nxt)

    def _state(self):
        return (self.tok, self.pos, self.finished, self.n_hard, self.n_steps, self.step_idx, self.out_tokens, self.out_len,
                self.hard_len, self.phase)

    @torch.no_grad()
    def generate(self, first_logits: torch.Tensor, max_new_tokens: int, *, temperature: float = 0.0, eos: int = -1,
                 use_graph: bool = True, check_every: int = 64, continuous: Optional[bool] = None, **filters):
        """Continues after :meth:`prefill`.  Returns tokens int64 [B, max_new_tokens]; a row's tokens end before its
        end-of-sequence token and are 0 from there on (``self.out_len`` holds each row's count).  With ``eos`` the
        loop looks every ``check_every`` steps whether all rows are done (the only host synchronisation).

        ``continuous`` (default: whenever the engine can): rows do not wait for each other's second latent iterations
        -- see :meth:`_generate_ticks`.  Greedy decoding gives the same tokens per row either way; sampled tokens come from
        the same per-row distributions but from other random draws (a tick draws for every row, a step once per token)."""
        if self.host_positions + max_new_tokens > self.max_len or self.host_hard_rows + max_new_tokens > self.max_hard:
            raise TahDuoError("generation would outgrow the KV slabs: construct the engine with a larger max_len / max_hard")
        dev = self.device
        greedy_fused = temperature <= 0.0 and self.fused_greedy and self.cfg.vocab % 8 == 0
        can_tick = self.can_run_continuous and self.fused_greedy and self.cfg.vocab % 8 == 0
        if continuous is None:
            continuous = can_tick and self.use_fused_glue and not self.measure_without_attention
        if continuous:
            if not can_tick:
                raise TahDuoError("continuous generation needs the fused attention and glue launches "
                                  "(at most 32 rows, 256 (row, kv head) pairs, slabs of at most 4096 rows)")
            return self._generate_ticks(first_logits, max_new_tokens, eos, use_graph and dev.type == "cuda",
                                        temperature=temperature, **filters)
        self.out_tokens.zero_()
        self.out_len.zero_()
        self.step_idx.zero_()
        first = self.sample(first_logits, temperature, **filters)
        if eos >= 0:
            self.finished |= first == eos
        keep = ~self.finished
        self.out_tokens[:, 0] = torch.where(keep, first, torch.zeros_like(first))
        self.out_len += keep.to(torch.int32)
        self.tok.copy_(first)
        self.step_idx += 1
        n = max_new_tokens - 1
        graph = self.capture(temperature, eos, **filters) if (use_graph and dev.type == "cuda" and n > 0) else None
        done = 0
        for i in range(n):
            if graph is not None:
                graph.replay()
            else:
                self._step_inplace(temperature, eos, **filters)
            done += 1
            if eos >= 0 and (i + 1) % check_every == 0 and bool(self.finished.all()):
                break
        self.host_positions += done
        self.host_hard_rows += done
        return self.out_tokens[:, :max_new_tokens]

    # ── rows at different latent iterations in one batch ─────────────────
    def _tick(self, parity: int, eos: int, limit: int, temperature: float = 0.0, **filters):
        """Every unfinished row advances by one latent iteration of its own token: the first iteration of its next
        token (phase 0), or the second iteration of the token whose first the previous tick ran (phase 1).  The
        logits go to ``self.logits2[parity]``; a row at phase 1 finds its first iteration's logits in the other one."""
        c, w, B = self.cfg, self.w, self.B
        ops.step_begin(self.tok, self.pos, self.finished, w.embed, self.cos, self.sin, x=self.x0, x_packed=self.xp,
                       cos_rows=self.cos_rows, sin_rows=self.sin_rows, slot=self.slot0, q_pos=self.qpos0, active=self.act,
                       phase=self.phase, x_alt=self.x1, hard_len=self.hard_len, q_depth=self.q_depth_rows,
                       append_at=self.append_at, eligible=self.eligible)
        self._pass_single_packed(self.x0, self.pos, None, self.slot0, self.qpos0, self.q_depth_rows, self.cos_rows,
                                 self.sin_rows, rows_packed=True)
        logits = ops.linear_rows(w.lm_head_p, self.xp, B, c.vocab, c.hidden, norm_eps=c.rms_eps, out=self.logits2[parity])
        if self.decider is not None:  # (rows at their second iteration are not eligible: what they left in hs_buf is not used)
            torch.logical_and(self._decide_rows(logits, self.hs_buf), self.eligible, out=self.hard)
        else:
            hr = ops.linear_rows(w.dec_w1_p, self.xp, B, c.decider_hidden, c.hidden, norm_eps=c.rms_eps, bias=w.dec_b1, relu=True)
            ops.decider_tail(hr, w.dec_w2.reshape(-1), w.dec_b2, w.threshold, hard=self.hard, active=self.eligible)
        ops.topk_mix(logits, w.embed, c.topk, row_enable=self.hard, out=self.x1)  # (other rows of x1 are not read)
        chosen = None
        if temperature > 0.0:
            # one draw per row from the final logits as the step-wise loop forms them (first iteration, plus the second
            # where there was one, summed in bf16); rows that only move on to their second iteration ignore theirs
            chosen = self._draw(logits, temperature, prev=self.logits2[1 - parity], add_prev=self.phase, **filters).contiguous()
        ops.greedy_tick(logits, self.logits2[1 - parity], eos, limit, hard_now=self.hard, phase=self.phase, tok=self.tok,
                        finished=self.finished, pos=self.pos, out_tokens=self.out_tokens, out_len=self.out_len,
                        hard_len=self.hard_len, n_hard=self.n_hard, n_steps=self.n_steps, chosen=chosen)

    def _launch_switches(self):
        """Every attribute that changes which kernels a captured step launches: part of both graph keys, so that
        flipping one between two generate() calls on the same prefill captures again instead of replaying a graph
        of the old path."""
        return (self.use_fused_glue, self.fused_greedy, self.fused_sampling, self.static_scratch, self.measure_without_attention, id(self.decider))

    def capture_ticks(self, eos: int, limit: int, temperature: float = 0.0, **filters):
        """The tick as two HIP graphs, one per logits buffer, after a warm-up tick whose state changes are undone."""
        key = (eos, limit, self.w.threshold, temperature, tuple(sorted(filters.items()))) + self._launch_switches()
        if self._tick_graphs is not None and self._tick_key == key:
            return self._tick_graphs
        state = [t.clone() for t in self._state()]
        lens = [sl.len.clone() for sl in self.slabs0 + self.slabs1]
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            self._tick(0, eos, limit, temperature, **filters)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        for t, old in zip(self._state(), state):
            t.copy_(old)
        for sl, ln in zip(self.slabs0 + self.slabs1, lens):
            sl.len.copy_(ln)
        graphs = []
        for parity in (0, 1):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._tick(parity, eos, limit, temperature, **filters)
            graphs.append(g)
        self._tick_graphs, self._tick_key = graphs, key
        return graphs

    def _generate_ticks(self, first_logits: torch.Tensor, max_new_tokens: int, eos: int, use_graph: bool, check_every: int = 8,
                        temperature: float = 0.0, **filters):
        """Generation in ticks.  The reference's loop (tah_model.py:580-706 inside utils.py:228-262) keeps the
        batch in step: every token costs the batch a first iteration and, if any row calls it hard, a second one --
        here a full pass over the weights for the one row in twelve that needs it.  Rows do not interact, so each row
        can run its own sequence of passes: a tick is one pass in which every row does the next iteration it needs.  A
        token costs its row 1 + [hard] ticks instead of 2, and the tokens are the ones the step-wise loop produces.
        The host looks every ``check_every`` ticks, once the fastest possible row could be done, whether all are."""
        B = self.B
        self.out_tokens.zero_()
        self.out_len.zero_()
        self.phase.zero_()
        first = self.sample(first_logits, temperature, **filters)
        if eos >= 0:
            self.finished |= first == eos
        keep = ~self.finished
        self.out_tokens[:, 0] = torch.where(keep, first, torch.zeros_like(first))
        self.out_len += keep.to(torch.int32)
        self.tok.copy_(first)
        limit = max_new_tokens
        reached = self.out_len >= limit
        self.finished |= reached
        n_min = max_new_tokens - 1
        graphs = self.capture_ticks(eos, limit, temperature, **filters) if (use_graph and n_min > 0) else None
        ticks = 0
        while n_min > 0:
            if graphs is not None:
                graphs[ticks % 2].replay()
            else:
                self._tick(ticks % 2, eos, limit, temperature, **filters)
            ticks += 1
            if ticks >= n_min and (ticks - n_min) % check_every == 0 and bool(self.finished.all()):
                break
            if ticks > 2 * n_min + check_every:
                raise TahDuoError("generation did not finish within two passes per token")
        self.ticks = ticks
        self.finished &= self.out_len < limit  # rows stopped by the limit have not ended
        self.host_positions += n_min
        self.host_hard_rows += n_min
        return self.out_tokens[:, :max_new_tokens]

    def capture(self, temperature: float = 0.0, eos: int = -1, **filters):
        """Captures one generation step in a HIP graph (after a warm-up step run on a side stream whose state
        changes are undone, so that library workspaces exist before the capture)."""
        key = (temperature, eos, tuple(sorted(filters.items()))) + self._launch_switches()
        if self._graph is not None and self._graph_key == key:
            return self._graph
        state = [t.clone() for t in self._state()]
        lens = [sl.len.clone() for sl in self.slabs0 + self.slabs1]
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            self._step_inplace(temperature, eos, **filters)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        # undo the warm-up step: state tensors and slab lengths (the rows it wrote lie beyond the lengths)
        for t, old in zip(self._state(), state):
            t.copy_(old)
        for sl, ln in zip(self.slabs0 + self.slabs1, lens):
            sl.len.copy_(ln)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._step_inplace(temperature, eos, **filters)
        self._graph, self._graph_key = g, key
        return g


def generate(engine: TaHDecodeEngine, tokenizer, model_inputs: dict, *, max_new_tokens: int = 1024, do_sample: bool = True,
             temperature: float = 1.0, top_p: float = 1.0, top_k: int = 0, min_p: float = 0.0, verbose: bool = False,
             use_graph: bool = True, **kwargs):
    """``TaHForCasualLM_generate`` (tah/model/utils.py:196-264) on the engine: same arguments (the engine in the
    model's place) and the same return value ``(output_tokens, generated_texts)`` -- per batch row the list of
    generated token ids up to, not including, the end-of-sequence token, and their decoded strings.

    ``model_inputs["input_ids"]`` (B, T) with an optional left-padding ``attention_mask``; the prompts are packed
    (pad tokens dropped) before the prefill.  Tokens are read back once, after the loop, not row by row per step
    (utils.py:243-245).  ``verbose`` (the reference prints every token coloured by its iteration count) is
    accepted and ignored."""
    del verbose, kwargs
    ids = model_inputs["input_ids"].to(engine.device)
    B, T = ids.shape
    if B != engine.B:
        raise TahDuoError(f"the engine was built for batch {engine.B}, got {B}")
    mask = model_inputs.get("attention_mask")
    valid = torch.ones_like(ids, dtype=torch.bool) if mask is None else mask.to(engine.device) != 0
    lens = valid.sum(1)
    cu = torch.cat([torch.zeros(1, dtype=lens.dtype, device=lens.device), lens.cumsum(0)]).to(torch.int32)
    first, _ = engine.prefill(ids[valid], cu)
    eos = tokenizer.eos_token_id if getattr(tokenizer, "eos_token_id", None) is not None else -1
    t = float(temperature) if do_sample else 0.0
    toks = engine.generate(first, max_new_tokens, temperature=t, eos=int(eos), use_graph=use_graph,
                           top_p=float(top_p), top_k=int(top_k), min_p=float(min_p))
    toks_h, len_h = toks.cpu(), engine.out_len.cpu()  # the one read-back
    out = [toks_h[b, : int(len_h[b])].tolist() for b in range(B)]
    return out, [tokenizer.decode(t_) if t_ else "" for t_ in out]
