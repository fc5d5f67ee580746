"""The learned iteration decider at inference, on the MI355X path.

``MLPIterDecider`` takes the place of ``tah.model.iter_decider.MLPIterDecider`` (iter_decider.py:193-301) when a model
is served: same constructor arguments, same parameter names (a state dict saved from the reference's class loads
with ``load_state_dict``), same ``forward(logits, iter_depth, all_hidden_states=None) -> (decision, decision_logits)``.
What changes is where the work is done:

* the only part that touches the vocabulary, ``torch.topk(logits, k).values`` (iter_decider.py:281: a sort-based
  selection over 151 936 logits per token), is one ``tah_topk_mix`` launch that writes the k largest logits of
  every row, largest first (``ops.topk_values``);
* the threshold is compared on the device: the reference reads it back with ``.item()`` on every call
  (iter_decider.py:296-298), which stalls the generation loop once per latent iteration.

* the dense layers behind it (iter_decider.py:128-190, :284-294), for the rows of a decode step (at most 32, bf16 layers,
  widths in multiples of 32), are a chain of ``tah_linear_rows`` launches, one per linear layer: a block's LayerNorm is
  folded into its first layer (scale into the weight, shift into the bias, the row's mean and deviation applied to the
  product), GELU is that launch's last step, the block's second layer and its ``dim_change`` are one product over the
  two inputs side by side (or the skip is the launch's residual), every layer writes the next one's operand in the
  order it is read in, and the concatenation of hidden states and projected logits is where the launches write.  Ten
  launches for the twelve linear layers (fifteen with the top-k values, two operand packs, sigmoid and compare) where
  the eager modules make about forty-five.  More rows (a prompt's tokens) and float32 copies
  of the decider go through the library's GEMMs.

Dropout is the identity here (inference); training the decider is the reference's own code's business.  Logits must be
bf16 (the kernel's type): anything else raises.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

STOP_LOGIT = -10.0  # decision logit reported once the iteration cap is reached (iter_decider.py:38, 273-274)
FUSED_MAX_ROWS = 32  # rows per call of the linear-layer kernel


def _ceil32(n: int) -> int:
    return (n + 31) // 32 * 32


class _FusedPlan:
    """The decider's dense layers as ``ops.linear_rows`` calls: weights re-ordered (LayerNorms folded in) once, the
    operand buffers the launches hand to each other, and the sequence of launches.  Every call on one decider writes the
    same buffers: calls follow each other on one stream (as a generation loop's do), they do not overlap."""

    def __init__(self, m: "MLPIterDecider", dev: torch.device):
        bf, f32 = torch.bfloat16, torch.float32
        H, S = m.hidden_states_size, max(1, len(m.hidden_states_layer_nums))
        self.kp = _ceil32(m.topk)
        z = lambda *shape: torch.zeros(*shape, dtype=bf, device=dev)
        self.top = z(FUSED_MAX_ROWS, self.kp)          # top-k values; the columns past topk stay zero
        self.top_p = z(32 * self.kp)
        self.comb_p = z(32 * (S + 1) * H)              # [hidden states | projected logits] as one packed operand
        self.feat_cols = S * H
        w = lambda lin: lin.weight.detach().to(dev, bf)
        b = lambda lin: lin.bias.detach().to(dev, f32)

        def layer(W, bias, **kw):
            n, k = W.shape
            return dict(w=ops.linear_pack_weight(W.contiguous()), n=n, k=k, bias=bias.to(bf).contiguous(), **kw)

        def behind_norm(W, bias, ln, **kw):  # W LayerNorm(x) + bias as one launch over x
            g, beta = ln.weight.detach().to(dev, f32), ln.bias.detach().to(dev, f32)
            Wf = (W.float() * g).to(bf)
            return layer(Wf, W.float() @ beta + bias, norm_eps=float(ln.eps), ln_colsum=Wf.float().sum(-1).contiguous(), **kw)

        Wlp = z(H, self.kp)
        Wlp[:, :m.topk] = w(m.logits_projection)
        self.logits_projection = layer(Wlp, b(m.logits_projection))
        self.combined = layer(w(m.combined_projection), b(m.combined_projection))
        self.x0_p = z(32 * self.combined["n"])
        bb = m.backbone
        self.input_projection = layer(w(bb["input_projection"]), b(bb["input_projection"]))
        self.blocks = []
        for blk in bb["blocks"]:
            up, down = blk["mlp"]["0"], blk["mlp"]["3"]
            wide, a = up.weight.shape
            first = behind_norm(w(up), b(up), blk["layer_norm"], gelu=True)
            if "dim_change" in blk:   # second layer and skip projection: one product over [h | x]
                second = layer(torch.cat([w(down), w(blk["dim_change"])], dim=1), b(down) + b(blk["dim_change"]))
            else:                     # the skip is the launch's residual: x row-major as well
                second = layer(w(down), b(down))
            # buf: h (the first layer's output) and behind it the block's input x, both packed
            self.blocks.append(dict(first=first, second=second, buf=z(32 * (wide + a)), h_cols=wide,
                                    x_rows=None if "dim_change" in blk else z(FUSED_MAX_ROWS, a)))
        out_ln, out_lin = bb["output_layer"]["0"], bb["output_layer"]["1"]
        last = out_lin.weight.shape[1]
        W16, b16 = z(16, last), torch.zeros(16, dtype=f32, device=dev)   # the one output column among a tile's sixteen
        W16[:1], b16[:1] = w(out_lin), b(out_lin)
        self.output = behind_norm(W16, b16, out_ln)
        self.last_p = z(32 * last)

    @staticmethod
    def supported(m: "MLPIterDecider") -> bool:
        """Every operand in whole steps of 32 columns, as the packed rows form holds them."""
        bb = m.backbone
        widths = [m.hidden_states_size, bb["input_projection"].weight.shape[0], bb["input_projection"].weight.shape[1]]
        for blk in bb["blocks"]:
            widths += list(blk["mlp"]["0"].weight.shape) + [blk["mlp"]["3"].weight.shape[0]]
        return all(x % 32 == 0 for x in widths) and bb["output_layer"]["1"].weight.shape[0] == 1

    @staticmethod
    def _run(L, x_packed, rows, **kw):
        return ops.linear_rows(L["w"], x_packed, rows, L["n"], L["k"], bias=L["bias"], norm_eps=L.get("norm_eps"),
                               ln_colsum=L.get("ln_colsum"), gelu=L.get("gelu", False), **kw)

    def decision_logits(self, rows: int) -> torch.Tensor:
        """From ``top[:rows]`` (the top-k features) and ``comb_p[: 32 * feat_cols]`` (the hidden states, packed) to the
        decision logits, bf16 [rows]."""
        run, blocks = self._run, self.blocks
        ops.linear_pack_rows(self.top[:rows], out=self.top_p)
        run(self.logits_projection, self.top_p, rows, out_packed=self.comb_p[32 * self.feat_cols:], want_out=False)
        run(self.combined, self.comb_p, rows, out_packed=self.x0_p, want_out=False)

        def hand_over(L, x_packed, i, **kw):  # a launch whose result is block i's input (or the output layer's)
            if i == len(blocks):
                return run(L, x_packed, rows, out_packed=self.last_p, want_out=False, **kw)
            x_rows = blocks[i]["x_rows"]
            run(L, x_packed, rows, out_packed=blocks[i]["buf"][32 * blocks[i]["h_cols"]:], want_out=x_rows is not None,
                out=None if x_rows is None else x_rows[:rows], **kw)

        hand_over(self.input_projection, self.x0_p, 0)
        for i, blk in enumerate(blocks):
            h_p, x_p = blk["buf"][:32 * blk["h_cols"]], blk["buf"][32 * blk["h_cols"]:]
            run(blk["first"], x_p, rows, out_packed=h_p, want_out=False)
            if blk["x_rows"] is None:
                hand_over(blk["second"], blk["buf"], i + 1)
            else:
                hand_over(blk["second"], h_p, i + 1, residual=blk["x_rows"][:rows])
        z16 = torch.empty(rows, 16, dtype=torch.bfloat16, device=self.top.device)
        run(self.output, self.last_p, rows, out=z16)
        return z16[:, 0]


def _named(**mods) -> nn.ModuleDict:
    return nn.ModuleDict(mods)


class MLPIterDecider(nn.Module):
    def __init__(self, topk: int = 100, hidden_states_size: int = 1024, hidden_states_layer_nums: Sequence[int] = (16, 20, 24, 28),
                 hidden_dims: Sequence[int] = (256, 512, 256), expansion_factor: int = 4, dropout_rate: float = 0.3,
                 normalize_input: bool = False, threshold: float = 0.5, max_iter: int = 3, dtype: torch.dtype = torch.bfloat16):
        super().__init__()
        del dropout_rate  # inference only
        self.topk, self.hidden_states_size, self.max_iter = int(topk), int(hidden_states_size), int(max_iter)
        self.hidden_states_layer_nums = [int(i) for i in hidden_states_layer_nums]
        self.normalize_input = bool(normalize_input)
        self.threshold = nn.Parameter(torch.tensor(threshold, dtype=dtype), requires_grad=False)
        slots = max(1, len(self.hidden_states_layer_nums))
        H, dims = self.hidden_states_size, [int(d) for d in hidden_dims]
        lin = lambda i, o: nn.Linear(i, o, dtype=dtype)
        if self.normalize_input:
            self.layer_norm_hidden_states = nn.LayerNorm(H * slots)
        self.logits_projection = lin(self.topk, H)
        self.combined_projection = lin(H * slots + H, dims[0])
        # backbone (iter_decider.py:131-190): a projection, residual blocks dims[i] -> dims[i + 1] (the last width once
        # more at the end), a final norm and a projection to one logit.  Children carry the names the reference's
        # Sequential / ModuleList give them, so that its state dict loads.
        widths = dims + [dims[-1]]
        blocks = []
        for a, b in zip(widths[:-1], widths[1:]):
            blk = _named(layer_norm=nn.LayerNorm(a, dtype=dtype), mlp=_named(**{"0": lin(a, a * expansion_factor), "3": lin(a * expansion_factor, b)}))
            if a != b:
                blk["dim_change"] = lin(a, b)
            blocks.append(blk)
        self.backbone = _named(input_projection=lin(dims[0], dims[0]), blocks=nn.ModuleList(blocks),
                               output_layer=_named(**{"0": nn.LayerNorm(dims[-1], dtype=dtype), "1": lin(dims[-1], 1)}))
        for m in self.backbone.modules():  # the reference's initialisation of the backbone (iter_decider.py:176-180)
            if isinstance(m, nn.Linear):
                nn.init.kaiming_normal_(m.weight)
                nn.init.zeros_(m.bias)
        self.fused_layers = True   # False: library GEMMs for every call
        self._plan, self._plan_key = None, None

    def fused_plan(self, dev: torch.device) -> "_FusedPlan":
        """The packed form of the dense layers on ``dev``, rebuilt when a parameter was written to since (a state dict
        loaded, a threshold calibrated).  A caller that captures graphs calls this once before capturing."""
        key = (str(dev),) + tuple((p.data_ptr(), p._version) for p in self.parameters())
        if self._plan is None or self._plan_key != key:
            with torch.no_grad():
                self._plan, self._plan_key = _FusedPlan(self, dev), key
        return self._plan

    def takes_fused_path(self, rows: int) -> bool:
        return (self.fused_layers and 0 < rows <= FUSED_MAX_ROWS and self.combined_projection.weight.dtype == torch.bfloat16
                and _FusedPlan.supported(self))

    # -- pieces ---------------------------------------------------------------------------------------------------
    def hidden_features(self, all_hidden_states: Optional[torch.Tensor], lead: Tuple[int, ...], like: torch.Tensor) -> torch.Tensor:
        """The configured layers of the stacked hidden states ``(..., L, H)`` (or ``(..., H)``: one layer) side by side,
        ``(*lead, n * H)``; zeros when there are none (iter_decider.py:244-263)."""
        slots = max(1, len(self.hidden_states_layer_nums))
        if all_hidden_states is None:
            return like.new_zeros(*lead, self.hidden_states_size * slots)
        hs = all_hidden_states if all_hidden_states.dim() == len(lead) + 2 else all_hidden_states.unsqueeze(-2)
        L = hs.size(-2)
        pick = self.hidden_states_layer_nums or [L - 1]
        if min(pick) < 0 or max(pick) >= L:
            raise ValueError(f"hidden_states_layer_nums {pick} out of range for {L} layers")
        # (plain slices side by side: indexing with a list would ship an index tensor to the device and wait for it)
        return torch.cat([hs[..., i, :] for i in pick], dim=-1).reshape(*lead, self.hidden_states_size * slots)

    def backbone_forward(self, x: torch.Tensor) -> torch.Tensor:
        b = self.backbone
        x = b["input_projection"](x)
        for blk in b["blocks"]:
            y = F.layer_norm(x, x.shape[-1:], blk["layer_norm"].weight, blk["layer_norm"].bias, blk["layer_norm"].eps)
            y = blk["mlp"]["3"](F.gelu(blk["mlp"]["0"](y)))
            x = (blk["dim_change"](x) if "dim_change" in blk else x) + y
        out = b["output_layer"]
        return out["1"](F.layer_norm(x, x.shape[-1:], out["0"].weight, out["0"].bias, out["0"].eps))

    # -- the decision -----------------------------------------------------------------------------------------------
    @torch.no_grad()
    def forward(self, logits: torch.Tensor, iter_depth: int, all_hidden_states: Optional[torch.Tensor] = None, **_) -> Tuple[torch.Tensor, torch.Tensor]:
        lead = tuple(logits.shape[:-1])
        if iter_depth >= self.max_iter:
            return self.decide_selected(logits, iter_depth, None)
        return self.decide_selected(logits, iter_depth, self.hidden_features(all_hidden_states, lead, logits))

    @torch.no_grad()
    def decide_selected(self, logits: torch.Tensor, iter_depth: int, feats: Optional[torch.Tensor]) -> Tuple[torch.Tensor, torch.Tensor]:
        """``forward`` for a caller that kept only the configured layers: ``feats`` ``(*lead, n * H)``, those layers' hidden
        states side by side in the configured order (what ``hidden_features`` returns)."""
        lead = tuple(logits.shape[:-1])
        if iter_depth >= self.max_iter:  # cap reached: nobody continues (iter_decider.py:273-274)
            return (torch.zeros(lead, dtype=torch.bool, device=logits.device),
                    torch.full(lead, STOP_LOGIT, dtype=logits.dtype, device=logits.device))
        if logits.dtype != torch.bfloat16:
            raise TypeError(f"MLPIterDecider: bf16 logits expected, got {logits.dtype} (the top-k kernel reads bf16; there is no other path)")
        flat = logits.reshape(-1, logits.size(-1))
        flat = flat if flat.stride(-1) == 1 else flat.contiguous()
        work = self.combined_projection.weight.dtype  # (bf16 as released; a float32 copy of the decider works too)
        rows = flat.size(0)
        if self.takes_fused_path(rows) and logits.size(-1) >= self.topk:
            plan = self.fused_plan(logits.device)
            feats = feats.reshape(rows, -1).to(work)
            if self.normalize_input:
                feats = self.layer_norm_hidden_states(feats.to(self.layer_norm_hidden_states.weight.dtype)).to(work)
                plan.top[:rows, :self.topk].copy_(torch.softmax(ops.topk_values(flat, self.topk), dim=-1))
            else:
                ops.topk_values(flat, self.topk, out=plan.top[:rows])
            ops.linear_pack_rows(feats.contiguous(), out=plan.comb_p[:32 * plan.feat_cols])
            decision_logits = plan.decision_logits(rows).view(lead)
            return torch.sigmoid(decision_logits) > self.threshold.to(decision_logits.dtype), decision_logits
        top = ops.topk_values(flat, self.topk).view(*lead, -1)
        feats, top = feats.to(work), top.to(work)
        if self.normalize_input:
            feats = self.layer_norm_hidden_states(feats.to(self.layer_norm_hidden_states.weight.dtype)).to(work)
            top = torch.softmax(top, dim=-1)
        x = self.combined_projection(torch.cat([feats, self.logits_projection(top)], dim=-1))
        decision_logits = self.backbone_forward(x).squeeze(-1)
        return torch.sigmoid(decision_logits) > self.threshold.to(decision_logits.dtype), decision_logits
