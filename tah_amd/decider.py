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

The small dense layers behind it stay library GEMMs.  Dropout is the identity here (inference); training the decider
is the reference's own code's business.  Logits must be bf16 (the kernel's type): anything else raises.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import ops

STOP_LOGIT = -10.0  # decision logit reported once the iteration cap is reached (iter_decider.py:38, 273-274)


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
        top = ops.topk_values(flat if flat.stride(-1) == 1 else flat.contiguous(), self.topk).view(*lead, -1)
        work = self.combined_projection.weight.dtype  # (bf16 as released; a float32 copy of the decider works too)
        feats, top = feats.to(work), top.to(work)
        if self.normalize_input:
            feats = self.layer_norm_hidden_states(feats.to(self.layer_norm_hidden_states.weight.dtype)).to(work)
            top = torch.softmax(top, dim=-1)
        x = self.combined_projection(torch.cat([feats, self.logits_projection(top)], dim=-1))
        decision_logits = self.backbone_forward(x).squeeze(-1)
        return torch.sigmoid(decision_logits) > self.threshold.to(decision_logits.dtype), decision_logits
