"""Kemavik: a layer-list decoder (``config.KemavikConfig``) whose norms sit on the sublayers'
OUTPUTS,

    x <- x + norm1(mixer(x));   x <- x + norm2(ff(x))   (the second only where the layer has a feed-forward)

with RMS norms whose weights are stored around zero (applied as ``1 + w``; the one is added
at load). The sublayers read the stream itself. Mixers (``models/mixers.py``): RWKV-style linear
attention with per-channel decays, or differential grouped-query attention with per-head query /
key norms; an attention layer may read an earlier layer's keys and values and then has no
cache of its own. Feed-forwards: dense with a squared ReLU, or a routed mixture of gated
experts (corrected top-k selection, identity experts, a shared expert).

The residual stream lives in 32-bit floats for every dtype. Each residual update is one fused
op (``add_normed``: the norm of the sublayer's output, the sum into the stream and the stream's
copy in the activation type that the next sublayer's projections read; after a mixture of experts
also the weighted combine of the experts' rows, the identity experts and the shared expert).
The linear attention reads the 32-bit stream directly.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from .layer_list import LayerListModel
from .mixers import RoutedMoE


class KemavikModel(LayerListModel):
    norm_offset = 1.0

    def forward(self, ids: torch.Tensor, meta, kv_caches) -> torch.Tensor:
        ops, cfg = self.ops, self.cfg
        state = meta.state
        if meta.id_src is not None:  # decode lookahead: row i's id is the previous step's sample tok[src[i]]
            src, tok = meta.id_src
            ids = torch.where(src >= 0, tok.index_select(0, src.clamp(min=0)), ids)
        h = F.embedding(ids, self.embed)
        residual = h.to(torch.float32, copy=True)
        for r, (i, _, _) in enumerate(self.runs):
            lw = self.layers[i]
            x = residual if getattr(lw.mixer, "input32", False) else h
            mix = lw.mixer.forward(x, meta, kv_caches[r], state[r] if state is not None else None)
            h = ops.add_normed(torch.empty_like(h), residual, mix, lw.norm1, cfg.norm_eps)
            if isinstance(lw.mlp, RoutedMoE):
                parts = lw.mlp.forward(h)
                h = ops.add_normed(torch.empty_like(h), residual, None, lw.norm2, cfg.norm_eps, parts)
            elif lw.mlp is not None:
                h = ops.add_normed(torch.empty_like(h), residual, lw.mlp.forward(h), lw.norm2, cfg.norm_eps)
            if self.capture is not None:
                self.capture.append(residual.clone())
        out = torch.empty_like(h)
        ops.scaled_add_group_rmsnorm(out, residual, self.final_norm, 1, cfg.norm_eps)
        return out
