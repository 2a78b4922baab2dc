"""``bench.py --layer-compare``: prefill and decode throughput of the layer-list decoders at
sizes that resemble a real model's layers, each beside the closest existing family at equal
size: Kesirax beside a Mixtral-style model (sliding-window attention + MoE feed-forward),
Fikizen beside a dense sliding-window model (grouped-query attention + gated dense
feed-forward), Kemavik beside Fikizen (the other design that mixes attention layers with
linear recurrences; its attention has no window), Topezen beside Kemavik (attention layers, a
matrix-valued recurrence and routed experts with a shared expert in both) and beside Kesirax (the
other design with latent attention). Random-init weights, synthetic prompts, a few layers of each (the per-layer
cost is what is compared). ``--layer-models`` picks the models; the ratios are given per pair.

Per size and model, through the engine's own scheduler and step function:
  prefill tok/s  = batch x prompt_len / time of the steps that compute the prompts
  decode tok/s   = batch x new_tokens / time of the decode steps that follow
One JSON line per (size, model) and a last line with the ratios.
"""
from __future__ import annotations

import json
import time

SIZES = {
    # name: width, heads, window, experts, top, ff, gru width, vocab
    "w1024": dict(width=1024, heads=8, window=512, experts=8, top=2, ff=512, gru=2048, vocab=32000, dense_ff=3072),
    "w2048": dict(width=2048, heads=16, window=1024, experts=16, top=2, ff=1024, gru=4096, vocab=32000, dense_ff=6144),
    "w4096": dict(width=4096, heads=32, window=1024, experts=8, top=2, ff=2048, gru=8192, vocab=32000, dense_ff=12288),
}


def kesirax_config(name, s):
    from ..config import HybridConfig, HybridLayerSpec, LatentAttentionSpec, MinGRUSpec, TableMoESpec

    attn = LatentAttentionSpec(heads=s["heads"], dim=128, rot_dim=64, vdim=128, q_rank=s["width"] // 2,
                               kv_rank=512, scale=192 ** -0.5, window=s["window"], rot_base=10000.0)
    ff = TableMoESpec(experts=s["experts"], top=s["top"], ff=s["ff"])
    layers = tuple(HybridLayerSpec(m, ff) for m in (attn, MinGRUSpec(s["gru"]), attn, MinGRUSpec(s["gru"])))
    return HybridConfig(name=f"kesirax-{name}", hidden_size=s["width"], vocab_size=s["vocab"], layers=layers,
                        norm_groups=4, max_position_embeddings=16384, eos_token_id=(2,), bos_token_id=1)


def mixtral_config(name, s):
    from ..config import ModelConfig

    return ModelConfig(name=f"mixtral-{name}", architecture="mixtral", family="mixtral", hidden_size=s["width"],
                       num_layers=4, num_heads=s["heads"], num_kv_heads=max(1, s["heads"] // 4), head_dim=128,
                       intermediate_size=s["ff"], vocab_size=s["vocab"], rope_theta=1e6,
                       max_position_embeddings=16384, num_experts=s["experts"], num_experts_per_tok=s["top"],
                       sliding_window=s["window"], layer_windows=(s["window"],) * 4, bos_token_id=1, eos_token_id=(2,))


def fikizen_config(name, s):
    """Four layers: gated sink attention + feed-forward, gated delta rule, attention beside the generalized
    delta rule + feed-forward, the first layer's weights once more."""
    from ..config import (DeltaRuleSpec, DenseFFSpec, FikizenConfig, GatedDeltaSpec, HybridLayerSpec,
                          ParallelMixerSpec, WindowAttentionSpec)

    H, kv = s["heads"], max(1, s["heads"] // 4)
    attn = dict(heads=H, kv_heads=kv, dim=128, vdim=128, scale=128 ** -0.5, window=s["window"], rot_dims=64,
                rot_base=5e5, sink=True)
    a = WindowAttentionSpec(gate=True, **attn)
    left = WindowAttentionSpec(bias=True, qk_norm=True, v_norm=True, **attn)
    par = ParallelMixerSpec(left, DeltaRuleSpec(heads=s["width"] // 64, dim=64, decay_rank=64), 0.75, 1.25)
    delta = GatedDeltaSpec(heads=H, kv_heads=kv, dim=128, vdim=128, conv=4)
    f = DenseFFSpec(s["dense_ff"])
    layers = (HybridLayerSpec(a, f), HybridLayerSpec(delta, None), HybridLayerSpec(par, f), HybridLayerSpec(a, f, 0))
    return FikizenConfig(name=f"fikizen-{name}", hidden_size=s["width"], vocab_size=s["vocab"], layers=layers,
                         logit_softcap=25.0, max_position_embeddings=16384, eos_token_id=(2,), bos_token_id=1)


def dense_config(name, s):
    """Four dense layers: sliding-window grouped-query attention + gated feed-forward whose three matrices
    hold as many weights as the two of the design beside it (2/3 of its inner size)."""
    from ..config import ModelConfig

    return ModelConfig(name=f"dense-{name}", architecture="llama", family="llama", hidden_size=s["width"],
                       num_layers=4, num_heads=s["heads"], num_kv_heads=max(1, s["heads"] // 4), head_dim=128,
                       intermediate_size=s["dense_ff"] * 2 // 3 // 256 * 256, vocab_size=s["vocab"], rope_theta=1e6,
                       max_position_embeddings=16384, sliding_window=s["window"], layer_windows=(s["window"],) * 4,
                       bos_token_id=1, eos_token_id=(2,))


def kemavik_config(name, s):
    """Four layers: decayed linear attention + dense feed-forward, differential attention + routed experts,
    differential attention on that layer's keys and values + dense feed-forward, linear attention + dense
    feed-forward. A differential head = two 64-dim maps over one 128-dim value head; plain causal attention."""
    from ..config import DenseFFSpec, HybridLayerSpec, KemavikConfig, RoutedMoESpec, WindowAttentionSpec, WkvSpec

    H, kv = s["heads"], max(1, s["heads"] // 4)
    attn = dict(heads=H, kv_heads=kv, dim=64, vdim=128, scale=64 ** -0.5, bias=True, out_bias=True, head_norm=True,
                maps=2, diff=0.6)
    wkv = WkvSpec(heads=s["width"] // 64, dim=64, decay_rank=64)
    d = DenseFFSpec(s["dense_ff"], "relu2")
    moe = RoutedMoESpec(experts=s["experts"], top=s["top"], ff=s["ff"], identity=2, scale=1.5, shared_ff=s["ff"])
    layers = (HybridLayerSpec(wkv, d), HybridLayerSpec(WindowAttentionSpec(**attn), moe),
              HybridLayerSpec(WindowAttentionSpec(kv_from=1, **attn), d), HybridLayerSpec(wkv, d))
    return KemavikConfig(name=f"kemavik-{name}", hidden_size=s["width"], vocab_size=s["vocab"], layers=layers,
                         max_position_embeddings=16384, eos_token_id=(2,), bos_token_id=1)


def topezen_config(name, s):
    """Four layers: latent attention + dense PolyNorm feed-forward, matrix memory + routed experts, capped window
    attention with kept first tokens and learned sinks + routed experts, matrix memory + dense feed-forward.
    Matrix memory heads as in large xLSTM models: key size width / 2 and value size width over width / 256 heads."""
    from ..config import (DenseFFSpec, HybridLayerSpec, LatentAttentionSpec, MLstmSpec, RoutedMoESpec, TopezenConfig,
                          WindowAttentionSpec)

    H, kv = s["heads"], max(1, s["heads"] // 4)
    latent = LatentAttentionSpec(heads=H, dim=128, rot_dim=64, vdim=128, q_rank=s["width"] // 2, kv_rank=512,
                                 scale=192 ** -0.5, rot_base=10000.0, interleaved=True, gate="channel")
    mem = MLstmSpec(heads=s["width"] // 256, dim=128, vdim=256, gate_cap=15.0)
    attn = WindowAttentionSpec(heads=H, kv_heads=kv, dim=128, vdim=128, scale=128 ** -0.5, window=s["window"],
                               keep_first=64, softcap=50.0, head_norm=True, sink=True, sink_weights=True)
    d = DenseFFSpec(s["dense_ff"], "polynorm")
    moe = RoutedMoESpec(experts=s["experts"], top=s["top"], ff=s["ff"], shared_ff=s["ff"], groups=4, keep_groups=2,
                        renorm=True)
    layers = (HybridLayerSpec(latent, d), HybridLayerSpec(mem, moe), HybridLayerSpec(attn, moe), HybridLayerSpec(mem, d))
    return TopezenConfig(name=f"topezen-{name}", hidden_size=s["width"], vocab_size=s["vocab"], layers=layers,
                         embed_scale=float(s["width"]) ** 0.5, max_position_embeddings=16384, eos_token_id=(2,),
                         bos_token_id=1)


MODELS = {"kesirax": kesirax_config, "mixtral": mixtral_config, "fikizen": fikizen_config, "dense": dense_config,
          "kemavik": kemavik_config, "topezen": topezen_config}
PAIRS = (("kesirax", "mixtral"), ("fikizen", "dense"), ("kemavik", "fikizen"), ("kemavik", "mixtral"),
         ("topezen", "kemavik"), ("topezen", "kesirax"))


def measure(mcfg, batch, prompt_len, new_tokens, device="cuda", repeats=2):
    import numpy as np
    import torch

    from ..config import EngineConfig
    from ..engine.llm_engine import LLMEngine
    from ..engine.request import SamplingParams
    from ..parallel.comm import TPGroup

    ecfg = EngineConfig(model=mcfg.name, load_format="dummy", device=device, max_num_seqs=max(batch, 8),
                        max_num_batched_tokens=8192, max_model_len=prompt_len + new_tokens + 8,
                        num_kv_blocks=(batch + 2) * (-(-(prompt_len + new_tokens + 8) // 16)) + 8,
                        enable_prefix_caching=False)
    tp = TPGroup(0, 1, None, torch.device("cuda", 0)) if device == "cuda" else TPGroup()
    eng = LLMEngine(ecfg, tp=tp, model_cfg=mcfg)
    rng = np.random.default_rng(0)
    sp = SamplingParams(temperature=0.0, max_tokens=new_tokens + 1, ignore_eos=True)

    def sync():
        if device == "cuda":
            torch.cuda.synchronize()

    best = {"prefill": 0.0, "decode": 0.0}
    for rep in range(repeats + 1):  # the first wave warms up
        seqs = [eng.add_request(None, rng.integers(3, mcfg.vocab_size, prompt_len).tolist(), sp) for _ in range(batch)]
        sync()
        t0 = time.perf_counter()
        while any(not s.output_token_ids or s.output_token_ids[-1] < 0 for s in seqs):
            eng.step()
        sync()
        t1 = time.perf_counter()
        while eng.has_unfinished():
            eng.step()
        sync()
        t2 = time.perf_counter()
        if rep:
            best["prefill"] = max(best["prefill"], batch * prompt_len / (t1 - t0))
            best["decode"] = max(best["decode"], batch * new_tokens / (t2 - t1))
    graphs = bool(eng.runner.use_graphs)
    eng.shutdown()
    del eng
    if device == "cuda":
        torch.cuda.empty_cache()
    return {"prefill_tok_s": round(best["prefill"], 1), "decode_tok_s": round(best["decode"], 1),
            "decode_graphs": graphs}


def main(args) -> int:
    sizes = [s for s in (args.layer_sizes.split(",") if args.layer_sizes else SIZES) if s]
    device = args.device
    out = []
    for name in sizes:
        s = SIZES[name]
        row = {"size": name, **s}
        models = [m for m in (args.layer_models or "kesirax,mixtral").split(",") if m]
        for label in models:
            cfg = MODELS[label](name, s)
            r = measure(cfg, args.layer_batch, args.layer_prompt, args.layer_new, device)
            row[label] = r
            print(json.dumps({"layer_compare": name, "model": cfg.name, "batch": args.layer_batch,
                              "prompt_len": args.layer_prompt, "new_tokens": args.layer_new, "dtype": "bf16",
                              "data": "synthetic", **r}), flush=True)
        for a, b in PAIRS:
            if a in row and b in row:
                row[f"{a}_vs_{b}"] = {k: round(row[a][f"{k}_tok_s"] / max(row[b][f"{k}_tok_s"], 1e-9), 3)
                                      for k in ("prefill", "decode")}
        if "kesirax_vs_mixtral" in row:
            row["prefill_ratio"] = row["kesirax_vs_mixtral"]["prefill"]
            row["decode_ratio"] = row["kesirax_vs_mixtral"]["decode"]
        out.append(row)
    keys = ("size", "prefill_ratio", "decode_ratio") + tuple(f"{a}_vs_{b}" for a, b in PAIRS)
    print(json.dumps({"layer_compare_summary": [{k: r[k] for k in keys if k in r} for r in out]}), flush=True)
    if args.out:
        with open(args.out, "w") as f:
            json.dump(out, f, indent=1)
    return 0
