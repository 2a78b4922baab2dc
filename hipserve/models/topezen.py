"""Topezen: a layer-list decoder (``config.TopezenConfig``) of parallel blocks with two norms and a
gate per channel on each sublayer's result,

    x <- x + sigmoid(rg1 h1 + b1) * mixer(h1) + sigmoid(rg2 h2 + b2) * ff(h2),   h1 = norm1(x), h2 = norm2(x)

(the second term only where the layer has a feed-forward). The RMS norms have one weight each; the
embedding is scaled. Mixers (``models/mixers.py``): causal latent attention (interleaved rotation,
per-channel output gate), an mLSTM matrix memory over state slots, or position-free grouped-query
attention with per-head query / key norms, capped scores, a window that keeps the first tokens
and a learned sink per head. Feed-forwards: dense with PolyNorm, or routed gated experts
(group-limited corrected top-k, renormalised weights, a shared expert).

The residual stream lives in 32-bit floats for every dtype. A whole block's residual update and
the NEXT block's two norms are one fused op (``gated_add_norms``: both gates' sigmoids, the
weighted combine of the experts' rows and the shared expert, the sum into the stream, one
root-mean-square for both norms); the gate projections ride on the sublayers' merged input GEMMs
(``mixers.attach_side``).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from .layer_list import LayerListModel
from .mixers import RoutedMoE, attach_side


class TopezenModel(LayerListModel):
    norm_library = "cell"

    def load_tensors(self, get):
        """Names as in ``LayerListModel.load_tensors``; ``l<i>.norm1`` / ``.norm2`` / ``final.norm`` hold one
        number each, and ``l<i>.rg1`` / ``.rg2`` (+ ``.b``) are the gates of the mixer's and the feed-forward's result."""
        dev, dt = self.device, self.dtype
        self.embed = get("embed").to(dev, dt).contiguous()
        self.lm_head = get("head").to(dev, dt).contiguous()
        self.final_norm = get("final.norm").to(dev, torch.float32).reshape(1)
        for i, lw in enumerate(self.layers):
            lw.norm1 = get(f"l{i}.norm1").to(dev, torch.float32).reshape(1)
            lw.mixer.load(get, f"l{i}.mix.")
            attach_side(lw.mixer, get(f"l{i}.rg1"))
            lw.b1 = get(f"l{i}.rg1.b").to(dev, torch.float32).contiguous()
            if lw.mlp is not None:
                lw.norm2 = get(f"l{i}.norm2").to(dev, torch.float32).reshape(1)
                lw.mlp.load(get, f"l{i}.mlp.")
                attach_side(lw.mlp, get(f"l{i}.rg2"))
                lw.b2 = get(f"l{i}.rg2.b").to(dev, torch.float32).contiguous()

    def random_tensors(self, seed: int = 0, std: float = 0.05) -> dict:
        cfg = self.cfg
        g = torch.Generator().manual_seed(seed)
        H, V = cfg.hidden_size, cfg.vocab_size
        out = {"embed": torch.randn(V, H, generator=g) / max(cfg.embed_scale, 1e-6), "head": torch.randn(V, H, generator=g) * std * 4,
               "final.norm": 1.0 + 0.1 * torch.randn((), generator=g)}
        for i, lw in enumerate(self.layers):
            out[f"l{i}.norm1"] = 1.0 + 0.1 * torch.randn((), generator=g)
            for k, v in lw.mixer.init_random(g, std).items():
                out[f"l{i}.mix.{k}"] = v
            out[f"l{i}.rg1"] = torch.randn(H, H, generator=g) * std * 2
            out[f"l{i}.rg1.b"] = torch.randn(H, generator=g) * 0.5
            if lw.mlp is not None:
                out[f"l{i}.norm2"] = 1.0 + 0.1 * torch.randn((), generator=g)
                for k, v in lw.mlp.init_random(g, std).items():
                    out[f"l{i}.mlp.{k}"] = v
                out[f"l{i}.rg2"] = torch.randn(H, H, generator=g) * std * 2
                out[f"l{i}.rg2.b"] = torch.randn(H, generator=g) * 0.5
        return {k: v.bfloat16().float() for k, v in out.items()}

    def step_workspace_bytes(self, tokens: int, seqs: int) -> int:
        return super().step_workspace_bytes(tokens, seqs) + tokens * self.cfg.hidden_size * 24

    # ---------------------------------------------------------------- forward
    def forward(self, ids: torch.Tensor, meta, kv_caches) -> torch.Tensor:
        ops, cfg = self.ops, self.cfg
        T, H = ids.shape[0], cfg.hidden_size
        state = meta.state
        if meta.id_src is not None:  # decode lookahead: row i's id is the previous step's sample tok[src[i]]
            src, tok = meta.id_src
            ids = torch.where(src >= 0, tok.index_select(0, src.clamp(min=0)), ids)
        residual = F.embedding(ids, self.embed).to(torch.float32, copy=True)
        if cfg.embed_scale != 1.0:
            residual *= cfg.embed_scale

        def norms_of(r):
            """The norm weights that read the stream after run r - 1: the next block's two, or the model's."""
            if r == len(self.runs):
                return self.final_norm, None
            lw = self.layers[self.runs[r][0]]
            return lw.norm1, (lw.norm2 if lw.mlp is not None else None)

        def outputs(w2):
            return (torch.empty(T, H, device=residual.device, dtype=self.dtype),
                    torch.empty(T, H, device=residual.device, dtype=self.dtype) if w2 is not None else None)

        w1, w2 = norms_of(0)
        h1, h2 = outputs(w2)
        ops.gated_add_norms(h1, h2, residual, w1, w2, cfg.norm_eps)
        for r, (i, _, _) in enumerate(self.runs):
            lw = self.layers[i]
            mix = lw.mixer.forward(h1, meta, kv_caches[r], state[r] if state is not None else None)
            first = (mix, lw.mixer.side_out, lw.b1)
            second = None
            if isinstance(lw.mlp, RoutedMoE):
                ye, pair_slot, _, wts, _, _, shared = lw.mlp.forward(h2)
                second = ((ye, pair_slot, wts, shared), lw.mlp.side_out, lw.b2)
            elif lw.mlp is not None:
                second = (lw.mlp.forward(h2), lw.mlp.side_out, lw.b2)
            w1, w2 = norms_of(r + 1)
            h1, h2 = outputs(w2)
            ops.gated_add_norms(h1, h2, residual, w1, w2, cfg.norm_eps, first, second)
            if self.capture is not None:
                self.capture.append(residual.clone())
        return h1
