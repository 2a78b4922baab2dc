"""Fikizen: a pre-norm layer-list decoder (``config.FikizenConfig``) on the hipserve op set.

    x <- x + mixer(norm1(x));   x <- x + ff(norm2(x))   (the second only where the layer has a feed-forward)

with the mixer one of ``models/mixers.py``: windowed sink attention with a per-head output
gate, a gated delta rule, or sink attention and a generalized delta rule side by side. A
layer may use another layer's weights; every layer RUN still has a paged cache and / or
state tensors of its own. The logits pass ``cap * tanh(. / cap)``.

The residual stream lives in 32-bit floats for every dtype; each residual update and the
norm that follows it are one fused op (``scaled_add_group_rmsnorm`` with one group). Per
engine step the model sees the flat token rows of all scheduled sequences (prompt portions
and single decode tokens alike); attention reads and writes the paged cache through the
step's block tables, the recurrences their sequences' state slots.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from .layer_list import LayerListModel


class FikizenModel(LayerListModel):
    # ---------------------------------------------------------------- forward
    def forward(self, ids: torch.Tensor, meta, kv_caches) -> torch.Tensor:
        ops, cfg = self.ops, self.cfg
        T, H = ids.shape[0], cfg.hidden_size
        state = meta.state
        if meta.id_src is not None:  # decode lookahead: row i's id is the previous step's sample tok[src[i]]
            src, tok = meta.id_src
            ids = torch.where(src >= 0, tok.index_select(0, src.clamp(min=0)), ids)
        residual = F.embedding(ids, self.embed).to(torch.float32, copy=True)
        h = torch.empty(T, H, device=residual.device, dtype=self.dtype)
        first = self.layers[self.runs[0][0]].norm1 if self.runs else self.final_norm
        ops.scaled_add_group_rmsnorm(h, residual, first, 1, cfg.norm_eps)
        for r, (i, _, _) in enumerate(self.runs):
            lw = self.layers[i]
            mix = lw.mixer.forward(h, meta, kv_caches[r], state[r] if state is not None else None)
            nxt = self.final_norm if r + 1 == len(self.runs) else self.layers[self.runs[r + 1][0]].norm1
            hn = torch.empty_like(h)
            if lw.mlp is not None:
                ops.scaled_add_group_rmsnorm(hn, residual, lw.norm2, 1, cfg.norm_eps, mix)
                ff = lw.mlp.forward(hn)
                hn = torch.empty_like(h)
                ops.scaled_add_group_rmsnorm(hn, residual, nxt, 1, cfg.norm_eps, ff)
            else:
                ops.scaled_add_group_rmsnorm(hn, residual, nxt, 1, cfg.norm_eps, mix)
            if self.capture is not None:
                self.capture.append(residual.clone())
            h = hn
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """32-bit logits = cap * tanh(head . hidden / cap)."""
        lg = super().compute_logits(hidden)
        cap = self.cfg.logit_softcap
        return torch.tanh(lg / cap) * cap if cap > 0 else lg
