"""Model and engine configuration.

``ModelConfig`` mirrors the fields of a HuggingFace ``config.json`` (Llama /
Mixtral families) and of GGUF ``llama.*`` metadata. ``EngineConfig`` carries the
flags the reference charts pass to the engine
(``vllm-models/helm-chart/templates/model-deployments.yaml:26-39``:
``--model --served-model-name --gpu-memory-utilization --tensor-parallel-size``)
plus the ``llama-server`` flags of the GGUF tier
(``ramalama-models/helm-chart/templates/model-deployments.yaml:26-35``).
Both are frozen after construction: no global mutable flags.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass, field


@dataclass(frozen=True)
class VisionConfig:
    """Qwen3-VL vision tower (HF ``vision_config``): a ViT over 16x16x2 (HxWxT)
    patches with a learned, bilinearly resampled position table, 2D RoPE, a 2x2
    spatial merger into the language model's hidden size and DeepStack features
    (merged outputs of intermediate blocks added to the first decoder layers)."""
    depth: int = 27
    hidden_size: int = 1152
    intermediate_size: int = 4304
    num_heads: int = 16
    patch_size: int = 16
    temporal_patch_size: int = 2
    in_channels: int = 3
    spatial_merge_size: int = 2
    out_hidden_size: int = 2048
    num_position_embeddings: int = 2304
    deepstack_visual_indexes: tuple = (8, 16, 24)
    hidden_act: str = "gelu_pytorch_tanh"
    # special tokens of the language model
    image_token_id: int = 151655
    video_token_id: int = 151656
    vision_start_token_id: int = 151652
    vision_end_token_id: int = 151653
    # image preprocessing (preprocessor_config.json)
    min_pixels: int = 65536
    max_pixels: int = 16777216
    image_mean: tuple = (0.5, 0.5, 0.5)
    image_std: tuple = (0.5, 0.5, 0.5)

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_heads

    @property
    def patch_dim(self) -> int:
        return self.in_channels * self.temporal_patch_size * self.patch_size ** 2

    @staticmethod
    def from_hf_dict(d: dict) -> "VisionConfig | None":
        v = d.get("vision_config")
        if not isinstance(v, dict) or "depth" not in v:
            return None
        kw = {k: v[k] for k in ("depth", "hidden_size", "intermediate_size", "num_heads", "patch_size",
                                "temporal_patch_size", "in_channels", "spatial_merge_size", "out_hidden_size",
                                "num_position_embeddings", "hidden_act") if k in v}
        kw["deepstack_visual_indexes"] = tuple(v.get("deepstack_visual_indexes") or ())
        for k in ("image_token_id", "video_token_id", "vision_start_token_id", "vision_end_token_id"):
            if d.get(k) is not None:
                kw[k] = int(d[k])
        return VisionConfig(**kw)


@dataclass(frozen=True)
class ModelConfig:
    name: str = "llama"
    architecture: str = "llama"          # llama | mixtral
    hidden_size: int = 4096
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 14336
    vocab_size: int = 128256
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: dict | None = None
    rope_mode: int = 0                    # 0 NeoX rotate-half (HF), 1 interleaved (GGUF)
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    num_experts: int = 0
    num_experts_per_tok: int = 0
    bos_token_id: int | None = 128000
    eos_token_id: tuple = (128001, 128009)
    # ---- family options (Qwen2/Qwen3/Qwen3-MoE/Gemma-3/Phi-3; defaults = Llama/Mixtral)
    family: str = "llama"                 # llama | mixtral | qwen2 | qwen3 | qwen3_moe | gemma3 | phi3
    qkv_bias: bool = False                # Qwen2: q/k/v projections carry a bias
    qk_norm: bool = False                 # Qwen3 / Gemma-3: per-head RMSNorm of q and k before RoPE
    moe_intermediate_size: int = 0        # expert width when it differs from intermediate_size (Qwen3-MoE)
    norm_topk_prob: bool = True           # renormalise the top-k routing weights (Mixtral: always)
    hidden_act: str = "silu"              # silu | gelu_tanh (Gemma GeGLU)
    sandwich_norm: bool = False           # Gemma-3: RMSNorm on the attention / MLP outputs too
    norm_offset: bool = False             # Gemma RMSNorm: x * (1 + w)
    embed_scale: float = 1.0              # Gemma: embeddings * sqrt(hidden)
    attn_scale: float = 0.0               # softmax scale (0 = 1/sqrt(head_dim)); Gemma: query_pre_attn_scalar^-0.5
    sliding_window: int = 0               # window of the sliding-attention layers (0 = none)
    layer_windows: tuple = ()             # per-layer window (0 = full attention); empty = all full
    rope_local_theta: float = 0.0         # RoPE base of the sliding layers (Gemma-3: 10000; 0 = rope_theta)
    partial_rotary_factor: float = 1.0
    # Qwen3-VL: interleaved multimodal RoPE (rotary pairs split T/H/W by this
    # section table; text tokens have t = h = w so it reduces to plain RoPE)
    mrope_section: tuple = ()
    vision: VisionConfig | None = None

    @property
    def expert_size(self):
        return self.moe_intermediate_size or self.intermediate_size

    def window_of(self, layer: int) -> int:
        return self.layer_windows[layer] if self.layer_windows else 0

    @property
    def q_size(self):
        return self.num_heads * self.head_dim

    @property
    def kv_size(self):
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        H, I, V, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_layers
        attn = H * (self.q_size + 2 * self.kv_size) + self.q_size * H
        if self.num_experts:
            mlp = 3 * H * self.expert_size * self.num_experts + H * self.num_experts
        else:
            mlp = 3 * H * I
        emb = V * H * (1 if self.tie_word_embeddings else 2)
        return L * (attn + mlp + 2 * H) + emb + H

    @staticmethod
    def from_hf_dict(d: dict, name: str = "model") -> "ModelConfig":
        """HF ``config.json`` -> ModelConfig for the served families. Multimodal
        wrappers (Gemma3ForConditionalGeneration, Qwen3-VL-MoE) contribute their
        ``text_config`` (the language model; vision towers are not served). Both the
        Hub's ``rope_theta``/``rope_scaling`` keys and the newer ``rope_parameters``
        form (per layer type for Gemma-3) are read."""
        arch = (d.get("architectures") or ["LlamaForCausalLM"])[0]
        mtype = d.get("model_type", "")
        vision = VisionConfig.from_hf_dict(d) if mtype.startswith("qwen3_vl") or "qwen3vl" in arch.lower() else None
        if isinstance(d.get("text_config"), dict):  # multimodal wrapper: the language model
            td = dict(d["text_config"])
            for k in ("eos_token_id", "bos_token_id", "tie_word_embeddings"):
                if k not in td and k in d:
                    td[k] = d[k]
            d = td
            mtype = d.get("model_type", mtype)
        family = _family_of(arch, mtype, d)
        nh = d["num_attention_heads"]
        H = d["hidden_size"]
        D = d.get("head_dim") or H // nh
        eos = d.get("eos_token_id", 2)
        eos = tuple(eos) if isinstance(eos, (list, tuple)) else (eos,)
        L = d["num_hidden_layers"]
        theta, scaling = _rope_params(d, "full_attention" if family == "gemma3" else None)
        kw = dict(
            name=name,
            architecture="mixtral" if family in ("mixtral", "qwen3_moe") else "llama",
            family=family,
            hidden_size=H,
            num_layers=L,
            num_heads=nh,
            num_kv_heads=d.get("num_key_value_heads") or nh,
            head_dim=D,
            intermediate_size=d["intermediate_size"],
            vocab_size=d["vocab_size"],
            rms_norm_eps=d.get("rms_norm_eps", 1e-5),
            rope_theta=theta,
            rope_scaling=scaling,
            max_position_embeddings=d.get("max_position_embeddings", 4096),
            tie_word_embeddings=d.get("tie_word_embeddings", family == "gemma3"),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=eos,
            partial_rotary_factor=float(d.get("partial_rotary_factor", 1.0) or 1.0),
        )
        if kw["partial_rotary_factor"] != 1.0:
            raise NotImplementedError("partial rotary embeddings are not supported")
        if vision is not None:
            rp = d.get("rope_parameters") or d.get("rope_scaling") or {}
            sec = tuple(int(x) for x in (rp.get("mrope_section") or (24, 20, 20)))
            if rp.get("mrope_interleaved") is False:
                raise NotImplementedError("non-interleaved MRoPE (Qwen2-VL layout) is not supported")
            kw.update(vision=vision, mrope_section=sec)
        if family == "mixtral":
            kw.update(num_experts=d.get("num_local_experts", 0) or 0,
                      num_experts_per_tok=d.get("num_experts_per_tok", 0) or 0)
        elif family == "qwen2":
            kw.update(qkv_bias=True)
        elif family == "qwen3":
            kw.update(qk_norm=True, qkv_bias=bool(d.get("attention_bias", False)))
        elif family == "qwen3_moe":
            if d.get("decoder_sparse_step", 1) != 1 or d.get("mlp_only_layers"):
                raise NotImplementedError("Qwen3-MoE with dense layers (decoder_sparse_step / mlp_only_layers)")
            kw.update(qk_norm=True, qkv_bias=bool(d.get("attention_bias", False)),
                      num_experts=d.get("num_experts") or d["num_local_experts"],
                      num_experts_per_tok=d["num_experts_per_tok"],
                      moe_intermediate_size=d["moe_intermediate_size"],
                      norm_topk_prob=bool(d.get("norm_topk_prob", False)))
        elif family == "gemma3":
            if d.get("final_logit_softcapping") or d.get("attn_logit_softcapping"):
                raise NotImplementedError("logit soft-capping (Gemma-2) is not supported")
            types = d.get("layer_types")
            if not types:
                pat = d.get("sliding_window_pattern", 6)
                types = ["sliding_attention" if (i + 1) % pat else "full_attention" for i in range(L)]
            win = int(d.get("sliding_window") or 0)
            local_theta, _ = _rope_params(d, "sliding_attention")
            kw.update(qk_norm=True, hidden_act="gelu_tanh", sandwich_norm=True, norm_offset=True,
                      embed_scale=float(H) ** 0.5,
                      attn_scale=float(d.get("query_pre_attn_scalar") or D) ** -0.5,
                      sliding_window=win,
                      layer_windows=tuple(win if t == "sliding_attention" else 0 for t in types),
                      rope_local_theta=local_theta)
        return ModelConfig(**kw)

    def replace(self, **kw) -> "ModelConfig":
        return dataclasses.replace(self, **kw)


def _family_of(arch: str, mtype: str, d: dict) -> str:
    a, t = arch.lower(), (mtype or "").lower()
    if t.startswith("qwen3_moe") or t.startswith("qwen3_vl_moe") or "qwen3moe" in a or "qwen3vlmoe" in a:
        return "qwen3_moe"
    if t.startswith("qwen3") or a.startswith("qwen3"):
        return "qwen3"
    if t.startswith("qwen2") or a.startswith("qwen2"):
        return "qwen2"
    if t.startswith("gemma3") or a.startswith("gemma3"):
        return "gemma3"
    if t == "phi3" or a.startswith("phi3"):
        return "phi3"
    if t == "mixtral" or "mixtral" in a or d.get("num_local_experts"):
        return "mixtral"
    if t in ("llama", "mistral", "") or "llama" in a or "mistral" in a:
        return "llama"
    raise NotImplementedError(f"unsupported architecture {arch!r} (model_type {mtype!r})")


_ROPE_TYPES = (None, "default", "llama3", "linear")


def _rope_params(d: dict, layer_type: str | None) -> tuple[float, dict | None]:
    """(theta, scaling) from the Hub keys (``rope_theta``, ``rope_scaling``,
    Gemma-3 ``rope_local_base_freq``) or the ``rope_parameters`` form (one dict,
    or one per layer type)."""
    rp = d.get("rope_parameters")
    if isinstance(rp, dict) and ("full_attention" in rp or "sliding_attention" in rp):
        rp = rp.get(layer_type or "full_attention")
    local = layer_type == "sliding_attention"
    if isinstance(rp, dict) and "rope_theta" in rp:
        theta = float(rp["rope_theta"])
        scaling = {k: v for k, v in rp.items() if k != "rope_theta"}
    elif local:  # Hub Gemma-3: local layers run plain RoPE on rope_local_base_freq
        theta, scaling = float(d.get("rope_local_base_freq", 10000.0)), None
    else:
        theta, scaling = float(d.get("rope_theta", 10000.0)), d.get("rope_scaling")
    if scaling is not None:
        typ = scaling.get("rope_type", scaling.get("type"))
        if typ not in _ROPE_TYPES:
            raise NotImplementedError(f"RoPE scaling {typ!r} is not supported ({', '.join(map(str, _ROPE_TYPES[1:]))})")
        if typ in (None, "default"):
            scaling = None
    return theta, scaling


_LLAMA3_SCALING = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                   "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}

# Public architecture hyper-parameters. Random-init weights of these
# shapes are what the benchmarks run (no network => no checkpoints).
PRESETS: dict[str, ModelConfig] = {
    "llama-3-8b": ModelConfig(name="llama-3-8b", hidden_size=4096, num_layers=32, num_heads=32,
                              num_kv_heads=8, intermediate_size=14336, vocab_size=128256,
                              rope_theta=500000.0, max_position_embeddings=8192),
    "llama-3.1-8b": ModelConfig(name="llama-3.1-8b", hidden_size=4096, num_layers=32, num_heads=32,
                                num_kv_heads=8, intermediate_size=14336, vocab_size=128256,
                                rope_theta=500000.0, rope_scaling=_LLAMA3_SCALING,
                                max_position_embeddings=131072),
    "llama-3-70b": ModelConfig(name="llama-3-70b", hidden_size=8192, num_layers=80, num_heads=64,
                               num_kv_heads=8, intermediate_size=28672, vocab_size=128256,
                               rope_theta=500000.0, max_position_embeddings=8192),
    "mixtral-8x7b": ModelConfig(name="mixtral-8x7b", architecture="mixtral", hidden_size=4096,
                                num_layers=32, num_heads=32, num_kv_heads=8,
                                intermediate_size=14336, vocab_size=32000, rope_theta=1e6,
                                max_position_embeddings=32768, num_experts=8,
                                num_experts_per_tok=2, bos_token_id=1, eos_token_id=(2,)),
    "tinyllama-1.1b": ModelConfig(name="tinyllama-1.1b", hidden_size=2048, num_layers=22,
                                  num_heads=32, num_kv_heads=4, head_dim=64,
                                  intermediate_size=5632, vocab_size=32000, rope_theta=10000.0,
                                  max_position_embeddings=2048, bos_token_id=1, eos_token_id=(2,)),
    # the reference chart's default model families (vllm-models/helm-chart/values.yaml:1-19,
    # ramalama-models/helm-chart/values.yaml:3-19), text models, public hyper-parameters
    "qwen3-0.6b": ModelConfig(name="qwen3-0.6b", family="qwen3", hidden_size=1024, num_layers=28,
                              num_heads=16, num_kv_heads=8, head_dim=128, intermediate_size=3072,
                              vocab_size=151936, rms_norm_eps=1e-6, rope_theta=1e6,
                              max_position_embeddings=40960, tie_word_embeddings=True, qk_norm=True,
                              bos_token_id=None, eos_token_id=(151643, 151645)),
    "qwen3-30b-a3b": ModelConfig(name="qwen3-30b-a3b", architecture="mixtral", family="qwen3_moe",
                                 hidden_size=2048, num_layers=48, num_heads=32, num_kv_heads=4, head_dim=128,
                                 intermediate_size=6144, moe_intermediate_size=768, num_experts=128,
                                 num_experts_per_tok=8, norm_topk_prob=True, vocab_size=151936,
                                 rms_norm_eps=1e-6, rope_theta=1e6, max_position_embeddings=40960,
                                 qk_norm=True, bos_token_id=None, eos_token_id=(151643, 151645)),
    # the reference's default HF model (vllm-models/helm-chart/values.yaml:8-12) with its
    # vision tower: Qwen3-VL-30B-A3B (text = Qwen3-30B-A3B with interleaved MRoPE)
    "qwen3-vl-30b-a3b": ModelConfig(name="qwen3-vl-30b-a3b", architecture="mixtral", family="qwen3_moe",
                                    hidden_size=2048, num_layers=48, num_heads=32, num_kv_heads=4, head_dim=128,
                                    intermediate_size=6144, moe_intermediate_size=768, num_experts=128,
                                    num_experts_per_tok=8, norm_topk_prob=True, vocab_size=151936,
                                    rms_norm_eps=1e-6, rope_theta=5e6, max_position_embeddings=262144,
                                    qk_norm=True, bos_token_id=None, eos_token_id=(151643, 151645),
                                    mrope_section=(24, 20, 20), vision=VisionConfig()),
    "gemma-3-27b": ModelConfig(name="gemma-3-27b", family="gemma3", hidden_size=5376, num_layers=62,
                               num_heads=32, num_kv_heads=16, head_dim=128, intermediate_size=21504,
                               vocab_size=262208, rms_norm_eps=1e-6, rope_theta=1e6,
                               rope_scaling={"rope_type": "linear", "factor": 8.0},
                               max_position_embeddings=131072, tie_word_embeddings=True, qk_norm=True,
                               hidden_act="gelu_tanh", sandwich_norm=True, norm_offset=True,
                               embed_scale=5376 ** 0.5, attn_scale=168 ** -0.5, sliding_window=1024,
                               layer_windows=tuple(1024 if (i + 1) % 6 else 0 for i in range(62)),
                               rope_local_theta=1e4, bos_token_id=2, eos_token_id=(1, 106)),
    "phi-3-mini": ModelConfig(name="phi-3-mini", family="phi3", hidden_size=3072, num_layers=32,
                              num_heads=32, num_kv_heads=32, head_dim=96, intermediate_size=8192,
                              vocab_size=32064, rope_theta=10000.0, max_position_embeddings=4096,
                              bos_token_id=1, eos_token_id=(32000, 32007)),
    # tiny shapes for CPU plumbing tests
    "tiny-llama": ModelConfig(name="tiny-llama", hidden_size=128, num_layers=2, num_heads=4,
                              num_kv_heads=2, head_dim=32, intermediate_size=256, vocab_size=512,
                              rope_theta=10000.0, max_position_embeddings=2048,
                              bos_token_id=1, eos_token_id=(2,)),
    # the 70B head layout in miniature (8 kv heads: one per rank at TP=8) for world-8 CPU runs
    "tiny-llama-tp8": ModelConfig(name="tiny-llama-tp8", hidden_size=256, num_layers=2, num_heads=16,
                                  num_kv_heads=8, head_dim=16, intermediate_size=512, vocab_size=512,
                                  rope_theta=500000.0, max_position_embeddings=2048,
                                  bos_token_id=1, eos_token_id=(2,)),
    "tiny-mixtral": ModelConfig(name="tiny-mixtral", architecture="mixtral", hidden_size=128,
                                num_layers=2, num_heads=4, num_kv_heads=2, head_dim=32,
                                intermediate_size=192, vocab_size=512, rope_theta=1e6,
                                max_position_embeddings=2048, num_experts=4,
                                num_experts_per_tok=2, bos_token_id=1, eos_token_id=(2,)),
    # GPU-test sized (head_dim 128 / 64 so the HIP kernels are exercised)
    "small-llama": ModelConfig(name="small-llama", hidden_size=512, num_layers=2, num_heads=8,
                               num_kv_heads=2, head_dim=64, intermediate_size=1024,
                               vocab_size=1024, rope_theta=10000.0, max_position_embeddings=4096,
                               bos_token_id=1, eos_token_id=(2,)),
    # long-context tests: Llama-3 head geometry (head_dim 128, GQA 4), 64K positions
    "small-llama-long": ModelConfig(name="small-llama-long", hidden_size=1024, num_layers=2, num_heads=8,
                                    num_kv_heads=2, head_dim=128, intermediate_size=2048,
                                    vocab_size=2048, rope_theta=500000.0, max_position_embeddings=65536,
                                    bos_token_id=1, eos_token_id=(2,)),
    "small-mixtral": ModelConfig(name="small-mixtral", architecture="mixtral", hidden_size=512,
                                 num_layers=2, num_heads=8, num_kv_heads=2, head_dim=64,
                                 intermediate_size=768, vocab_size=1024, rope_theta=1e6,
                                 max_position_embeddings=4096, num_experts=8,
                                 num_experts_per_tok=2, bos_token_id=1, eos_token_id=(2,)),
}


def preset_key(model: str) -> str | None:
    """Built-in preset a model name / Hub id maps to (``meta-llama/Meta-Llama-3-8B``
    -> ``llama-3-8b``), or None. Local paths never map to a preset."""
    if os.path.exists(model):
        return None
    key = model.lower().split("/")[-1]
    for k in PRESETS:
        if key == k or key.replace("meta-", "").replace("-instruct", "") == k:
            return k
    return None


def resolve_model_config(model: str, name: str | None = None) -> ModelConfig:
    """Preset name, HF model directory (config.json), HF cache id, or a .gguf file.
    (A Hub id is first materialised into the cache by ``weights.hub.materialize``.)"""
    k = preset_key(model)
    if k is not None and not _hf_cache_dir(model):
        return PRESETS[k]
    if os.path.isdir(model) and os.path.exists(os.path.join(model, "config.json")):
        with open(os.path.join(model, "config.json")) as f:
            cfg = config_from_dict(json.load(f), name=name or os.path.basename(os.path.normpath(model)))
            return _with_preprocessor(cfg, model) if isinstance(cfg, ModelConfig) else cfg
    if model.endswith(".gguf") and os.path.exists(model):
        from .weights.gguf import GGUFFile

        return GGUFFile(model).model_config(name=name)
    hub = _hf_cache_dir(model)
    if hub:
        with open(os.path.join(hub, "config.json")) as f:
            return _with_preprocessor(ModelConfig.from_hf_dict(json.load(f), name=name or model), hub)
    raise ValueError(f"unknown model {model!r}: not a preset ({', '.join(PRESETS)}), "
                     "a directory with config.json, a cached HF id or a .gguf file")


def _with_preprocessor(cfg: ModelConfig, path: str) -> ModelConfig:
    """Image preprocessing limits of a vision model from its preprocessor_config.json
    (``size.shortest_edge`` / ``longest_edge`` or ``min_pixels`` / ``max_pixels``,
    ``image_mean`` / ``image_std``)."""
    p = os.path.join(path, "preprocessor_config.json")
    if cfg.vision is None or not os.path.exists(p):
        return cfg
    with open(p) as f:
        d = json.load(f)
    size = d.get("size") or {}
    kw = {}
    lo = d.get("min_pixels") or size.get("shortest_edge") or size.get("min_pixels")
    hi = d.get("max_pixels") or size.get("longest_edge") or size.get("max_pixels")
    if lo:
        kw["min_pixels"] = int(lo)
    if hi:
        kw["max_pixels"] = int(hi)
    for k in ("image_mean", "image_std"):
        if d.get(k):
            kw[k] = tuple(float(x) for x in d[k])
    if d.get("patch_size") and int(d["patch_size"]) != cfg.vision.patch_size:
        raise ValueError("preprocessor patch_size differs from the vision tower's")
    return cfg.replace(vision=dataclasses.replace(cfg.vision, **kw))


def _hf_cache_dir(repo_id: str) -> str | None:
    """Locate a snapshot of an HF Hub repo in the local cache (offline): the
    revision ``refs/main`` names (what the Hub client resolved last), else the most
    recently written snapshot that has a config.json."""
    if "/" not in repo_id:
        return None
    home = os.environ.get("HF_HOME", os.path.expanduser("~/.cache/huggingface"))
    repo = os.path.join(home, "hub", "models--" + repo_id.replace("/", "--"))
    base = os.path.join(repo, "snapshots")
    if not os.path.isdir(base):
        return None
    try:
        with open(os.path.join(repo, "refs", "main")) as f:
            ref = f.read().strip()
    except OSError:
        ref = ""
    if ref and os.path.exists(os.path.join(base, ref, "config.json")):
        return os.path.join(base, ref)
    snaps = [os.path.join(base, s) for s in os.listdir(base)]
    snaps = [p for p in snaps if os.path.exists(os.path.join(p, "config.json"))]
    return max(snaps, key=lambda p: (os.path.getmtime(p), p)) if snaps else None


GGUF_QUANTS = ("q4_k_m", "q8_0", "q4_0")


def default_batched_tokens(model: str, load_format: str = "auto", quantization: str | None = None) -> int:
    """Prefill token budget per step when none is given: 8192; 16384 for GGUF weights and
    32768 for INT8 weight-only ones. Both keep only their quantised weights and dequantise
    each projection (every expert, for MoE) into a bf16 scratch once per prefill step, a
    cost that more tokens per step spread thinner:
      * Llama-3-8B Q4_K_M: 7,726 -> 8,044 tok/s, p50 TTFT 482 -> 530 ms
        (profiles/r5_bench_q4km_chunk8k.json, r5_bench_q4km_chunk16k.json);
      * Qwen3-30B-A3B INT8 (experts dequantised into the one-launch grouped GEMM's packed
        layout): 4,134 / 646 ms (8K) -> 4,380 / 570 (16K) -> 4,531 / 570 (32K) with a separate
        pack pass, 4,666 / 490 (32K) dequantising straight into the layout; above the
        4,155 / 623 ms of bf16 prefill shadows at 8K with 34 % more KV blocks
        (profiles/r5_bench_q3int8_packed_moe_*.json, r5_bench_q3int8_shadows.json).
    FP8 keeps 8192 (Gemma-3-27B: 2,839 vs 2,854 tok/s at 16K, TTFT 1,110 vs 1,186 ms), and
    so do bf16 MoE models (Mixtral-8x7B: 1,648 / 1,655 / 1,675 tok/s at 8K / 16K / 32K for
    TTFT 558 / 616 / 753 ms, profiles/r5_bench_mixtral*.json). A larger budget also
    lengthens the decode stall of running requests during a prefill step: latency-bound
    deployments pass a smaller --max-num-batched-tokens.
    bf16 models keep 8192: 16384 gave the same 7,730 tok/s at 480 vs 434 ms TTFT and 4096
    7,607 / 432 ms (profiles/r5_bench_8b_chunk16k.json, r5_bench_8b_chunk4k.json)."""
    if quantization is None:
        quantization = checkpoint_quantization(model)
    if quantization == "int8":
        return 32768
    gguf = quantization in GGUF_QUANTS or load_format == "gguf" or str(model).lower().endswith(".gguf")
    return 16384 if gguf else 8192


def checkpoint_quantization(model: str) -> str | None:
    """"int8" / "fp8" from a local HF checkpoint's ``quantization_config`` (compressed-
    tensors weight groups, AWQ / GPTQ bits), else None (presets, Hub ids not yet
    downloaded: the caller's default applies)."""
    path = os.path.join(str(model), "config.json")
    if not os.path.isfile(path):
        return None
    try:
        with open(path) as f:
            q = json.load(f).get("quantization_config") or {}
    except (OSError, ValueError):
        return None
    method = str(q.get("quant_method", "")).lower()
    if method == "fp8":
        return "fp8"
    if method in ("awq", "gptq"):
        return "int8" if int(q.get("bits", 0)) == 8 else None
    for grp in (q.get("config_groups") or {}).values():
        w = (grp or {}).get("weights") or {}
        if int(w.get("num_bits", 0)) == 8:
            return "fp8" if str(w.get("type", "")).lower() == "float" else "int8"
    return None


# --kv-cache-dtype values (vLLM's spellings) -> element kind
KV_CACHE_DTYPES = {"auto": "auto", "bf16": "auto", "bfloat16": "auto", "fp8": "fp8", "fp8_e4m3": "fp8"}


@dataclass(frozen=True)
class EngineConfig:
    model: str = "llama-3-8b"
    served_model_name: str | None = None
    tokenizer: str | None = None
    load_format: str = "auto"            # auto | dummy | safetensors | gguf
    dtype: str = "bfloat16"
    device: str = "cuda"
    tensor_parallel_size: int = 1
    gpu_memory_utilization: float = 0.90
    max_model_len: int | None = None
    block_size: int = 16
    max_num_seqs: int = 256
    max_num_batched_tokens: int = 8192
    num_kv_blocks: int | None = None     # override the memory-derived KV pool size
    enable_prefix_caching: bool = True
    enforce_eager: bool = False
    cuda_graph_max_bs: int = 256
    seed: int = 0
    trust_remote_code: bool = False
    decode_partition: int = 512
    # paged KV cache element: "auto" (= the activation dtype, bf16) or "fp8" / "fp8_e4m3"
    # (OCP e4m3, per-tensor scale 1 as vLLM's --kv-cache-dtype fp8 without calibrated
    # scales: half the KV bytes per token, so 2x the KV blocks and half the decode
    # attention's HBM stream; K / V are rounded to e4m3 when written)
    kv_cache_dtype: str = "auto"
    host: str = "0.0.0.0"
    port: int = 8080
    extra: dict = field(default_factory=dict)

    def __post_init__(self):
        # the attention kernels index the paged cache with shifts / masks
        b = self.block_size
        if b < 16 or b > 256 or b & (b - 1):
            raise ValueError(f"block_size must be a power of two in [16, 256], got {b}")
        if self.kv_cache_dtype not in KV_CACHE_DTYPES:
            raise ValueError(f"kv_cache_dtype must be one of {sorted(KV_CACHE_DTYPES)}, got {self.kv_cache_dtype!r}")

    @property
    def kv_fp8(self) -> bool:
        return KV_CACHE_DTYPES[self.kv_cache_dtype] == "fp8"

    def replace(self, **kw) -> "EngineConfig":
        return dataclasses.replace(self, **kw)

    @property
    def model_name(self) -> str:
        return self.served_model_name or self.model


# ---------------------------------------------------------------------------------
# Layer-list ("hybrid") decoders: the config file lists the layers one by one, each
# with its sequence mixer and its feed-forward, instead of one repeated block.

@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention through low-rank latents: queries go through a ``q_rank`` latent, keys
    and values are expanded per head from one ``kv_rank`` latent per token, and a
    ``rot_dim`` rotary key part is shared by all heads. Only the latent and the rotary
    key part are cached. ``window`` 0 = plain causal attention. ``interleaved``: the rotation
    pairs coordinate 2i with 2i + 1 (else i with i + rot_dims / 2). ``gate``: ``head`` multiplies
    head h's output by sigmoid of one number per head, ``channel`` multiplies the concatenated
    heads element by element by sigmoid of a projection of that size, ``none`` has no gate."""
    heads: int
    dim: int            # unrotated query/key dims per head
    rot_dim: int        # rotated query/key dims per head (one shared key part)
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int = 0
    rot_base: float = 10000.0
    rot_dims: int = 0   # leading dims of the rotated part that are rotated (0 = all of rot_dim)
    interleaved: bool = False
    gate: str = "head"

    kind = "latent_attention"

    @property
    def key_dim(self) -> int:
        """Cached elements per token."""
        return self.kv_rank + self.rot_dim

    @property
    def gate_size(self) -> int:
        """Rows of the gate projection."""
        return {"head": self.heads, "channel": self.heads * self.vdim, "none": 0}[self.gate]


@dataclass(frozen=True)
class MinGRUSpec:
    """Gated linear recurrence whose gates read only the current token (minGRU)."""
    width: int

    kind = "mingru"


@dataclass(frozen=True)
class TableMoESpec:
    """Mixture of small feed-forwards whose experts are looked up per token id in a
    table (no learned router at run time); every chosen expert weighs 1 / top."""
    experts: int
    top: int
    ff: int

    kind = "moe"


@dataclass(frozen=True)
class WindowAttentionSpec:
    """Grouped-query attention over a sliding window (``window`` keys: the token itself and
    the ``window - 1`` before it; 0 = plain causal) with rotate-half rotary positions on the
    first ``rot_dims`` dims of every head. Options, each independent of the others:
    ``sink`` adds one to the softmax denominator (a key of score 0 without a value), with
    ``sink_weights`` exp of a learned number per head instead of one,
    ``softcap`` > 0 passes the scaled scores through ``softcap * tanh(. / softcap)``,
    ``keep_first`` > 0 keeps the sequence's first ``keep_first`` tokens visible behind the window,
    ``gate`` multiplies head h's output by sigmoid of a per-head projection of the mixer input,
    ``bias`` adds biases in the q / k / v projections, ``qk_norm`` applies a weighted RMS norm
    over the WHOLE q (and k) projection before the rotation, ``head_norm`` one over every
    query / key head with a weight of ``dim`` elements that all heads share, ``v_norm`` divides
    every value head by its root mean square (cached so), ``out_bias`` adds a bias in the
    output projection.

    ``maps`` = 2 is differential attention: every query head and every key head carries two
    maps side by side ([map 1 | map 2], ``dim`` each); each map is a softmax attention of its
    own over the same values, and the head's output is ``a1 - lam * a2`` divided by its root
    mean square, times ``1 - diff`` (``lam`` comes from learned vectors and ``diff``).
    ``kv_from`` = j: the layer has no key / value projections and reads layer j's cache."""
    heads: int
    kv_heads: int
    dim: int            # query / key dims per head
    vdim: int           # value dims per head
    scale: float
    window: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    sink: bool = False
    gate: bool = False
    bias: bool = False
    qk_norm: bool = False
    v_norm: bool = False
    head_norm: bool = False
    out_bias: bool = False
    maps: int = 1
    diff: float = 0.0
    kv_from: int | None = None
    softcap: float = 0.0
    keep_first: int = 0
    sink_weights: bool = False

    kind = "attention"

    @property
    def q_size(self) -> int:
        return self.heads * self.maps * self.dim

    @property
    def k_size(self) -> int:
        return self.kv_heads * self.maps * self.dim

    @property
    def v_size(self) -> int:
        return self.kv_heads * self.vdim

    @property
    def cache_dim(self) -> int:
        """Cached elements per token: all key heads, then all value heads (none when the layer
        reads another layer's cache)."""
        return 0 if self.kv_from is not None else self.k_size + self.v_size


@dataclass(frozen=True)
class WkvSpec:
    """Linear attention with a decay per key channel and token (RWKV-style time mixing): every
    projection reads its own blend of the token's and the previous token's input, the decay
    comes from a ``decay_rank`` bottleneck, the current token enters its own read-out through a
    bonus vector, and the per-head ``dim x dim`` state is 32-bit."""
    heads: int
    dim: int
    decay_rank: int = 0     # read from the checkpoint when 0

    kind = "wkv"

    @property
    def size(self) -> int:
        return self.heads * self.dim


@dataclass(frozen=True)
class GatedDeltaSpec:
    """Gated delta rule: per head a ``dim x vdim`` state that decays by one number per token
    and is corrected towards the token's value along its unit key; q, k and v pass a causal
    convolution of ``conv`` taps and SiLU first. ``kv_heads`` query / key heads serve ``heads``
    value heads."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    kind = "delta"

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    @property
    def proj_size(self) -> int:
        """Merged input projection: q | k | v | beta | decay | output gate."""
        return self.conv_channels + 2 * self.heads + self.heads * self.vdim


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Generalized delta rule: per head a ``dim x dim`` state with a decay and a removal rate
    per key channel; the decay comes from a ``decay_rank`` bottleneck."""
    heads: int
    dim: int
    decay_rank: int = 0     # read from the checkpoint when 0

    kind = "delta_rule"

    @property
    def size(self) -> int:
        return self.heads * self.dim


@dataclass(frozen=True)
class MLstmSpec:
    """Matrix memory (mLSTM): per head a ``dim x vdim`` state S and a normaliser n of ``dim``
    elements, written with an exponential input gate and decayed by a sigmoid forget gate, both
    one number per head and token and both capped, ``cap * tanh(. / cap)``, before their
    non-linearity; a running maximum m of the log gates keeps the exponentials bounded. The
    read-out ``S^T q / (max(|n . q|, exp(-m)) + 1e-6)`` is divided by its per-head root mean
    square, weighted and gated by a sigmoid of a projection of the input."""
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    kind = "mlstm"

    @property
    def out_size(self) -> int:
        return self.heads * self.vdim


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers on the same input, their outputs summed with fixed weights."""
    left: object
    right: object
    left_scale: float = 1.0
    right_scale: float = 1.0

    kind = "parallel"


@dataclass(frozen=True)
class DenseFFSpec:
    """down(act(up(x))) with one of the op set's elementwise activations (``xielu``, ``relu2``) or
    ``polynorm``: a N(z) + b N(z^2) + c N(z^3) + e with four learned numbers, N dividing a token's
    vector by its root mean square."""
    ff: int
    act: str = "xielu"

    kind = "dense"


@dataclass(frozen=True)
class RoutedMoESpec:
    """Mixture of gated feed-forwards with a learned softmax router: the ``top`` experts with
    the largest score + correction are chosen, weighted by their (uncorrected, not
    renormalised) score times ``scale``. The last ``identity`` router outputs are experts
    without weights that return their input; ``shared_ff`` > 0 adds a gated feed-forward that
    every token runs. ``groups`` > 1: the router outputs form that many equal groups of
    neighbours, a group scores the largest corrected score in it, and only the experts of the
    ``keep_groups`` best groups can be chosen. ``renorm``: the chosen scores are divided by
    their sum before the scaling."""
    experts: int
    top: int
    ff: int
    identity: int = 0
    scale: float = 1.0
    shared_ff: int = 0
    groups: int = 1
    keep_groups: int = 1
    renorm: bool = False

    kind = "routed_moe"


@dataclass(frozen=True)
class HybridLayerSpec:
    mixer: object               # a mixer spec of this section
    mlp: object | None          # TableMoESpec | DenseFFSpec | None
    weights_of: int | None = None   # the layer whose weights this one uses (its own when None)


@dataclass(frozen=True)
class HybridConfig:
    """A decoder given as a list of layers (``layers[i]``), of which the span
    ``loop_start .. loop_stop - 1`` runs ``loop_times`` times in a row with the same
    weights. Carries the attributes the engine reads from any model config."""
    name: str = "hybrid"
    architecture: str = "kesirax"
    family: str = "kesirax"
    hidden_size: int = 256
    vocab_size: int = 512
    layers: tuple = ()
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-6
    norm_groups: int = 1
    logit_scale: float = 1.0
    max_position_embeddings: int = 1 << 20   # rotary angles are computed, not tabulated
    default_model_len: int = 32768            # context length served when --max-model-len is not given
    bos_token_id: int | None = None
    eos_token_id: tuple = ()
    vision: object = None
    num_experts: int = 0                      # no learned-router MoE (engine start-up tuning keys on it)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """Layer runs in execution order: (layer index, pass index, starts_pass) where
        ``starts_pass`` marks the first layer of every pass of the loop but the first."""
        a, b, n = self.loop_start, self.loop_stop, self.loop_times
        out = [(i, 0, False) for i in range(0, a)]
        for t in range(n if b > a else 0):
            out += [(i, t, t > 0 and i == a) for i in range(a, b)]
        out += [(i, 0, False) for i in range(b if b > a else a, len(self.layers))]
        return out

    def num_params(self) -> int:
        H, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        for l in self.layers:
            m = l.mixer
            if isinstance(m, LatentAttentionSpec):
                n += H * (m.q_rank + m.key_dim + m.heads) + m.q_rank * m.heads * (m.dim + m.rot_dim)
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + m.heads * m.vdim * H
            else:
                n += 4 * H * m.width
            if l.mlp is not None:
                n += 2 * l.mlp.experts * l.mlp.ff * H
        return n

    def replace(self, **kw) -> "HybridConfig":
        return dataclasses.replace(self, **kw)

    @staticmethod
    def from_dict(d: dict, name: str = "model") -> "HybridConfig":
        layers = []
        for l in d["layers"]:
            m = l["mixer"]
            if l["type"] == "latent_attention":
                rot = m.get("rot") or {}
                mixer = LatentAttentionSpec(
                    heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                    q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                    window=int((m.get("mask") or {}).get("size") or 0),
                    rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims") or m["rot_dim"]))
            elif l["type"] == "mingru":
                mixer = MinGRUSpec(width=int(m["width"]))
            else:
                raise NotImplementedError(f"unknown mixer {l['type']!r}")
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") != "moe":
                    raise NotImplementedError(f"unknown feed-forward {f.get('kind')!r}")
                mlp = TableMoESpec(experts=int(f["router"]["experts"]), top=int(f["router"]["top"]),
                                   ff=int(f["expert"]["ff"]))
            layers.append(HybridLayerSpec(mixer, mlp))
        lp = d.get("loop") or {}
        norm = d.get("norm") or {}
        eos = d.get("eos_token_id", ())
        eos = tuple(eos) if isinstance(eos, (list, tuple)) else (eos,)
        return HybridConfig(
            name=name, hidden_size=int(d["width"]), vocab_size=int(d["vocab"]), layers=tuple(layers),
            loop_start=int(lp.get("start", 0)), loop_stop=int(lp.get("stop", 0)), loop_times=int(lp.get("times", 1)),
            norm_eps=float(norm.get("eps", 1e-6)), norm_groups=int(norm.get("groups", 1)),
            logit_scale=float(d.get("logit_scale", 1.0)), bos_token_id=d.get("bos_token_id"), eos_token_id=eos)


@dataclass(frozen=True)
class FikizenConfig:
    """Fikizen: a pre-norm decoder given as a list of layers, each with one mixer (windowed
    sink attention with an output gate, a gated delta rule, or attention and a generalized
    delta rule in parallel) and an optional dense feed-forward. A layer can use another
    layer's weights (``weights_of``) with a cache / state of its own. Logits are soft-capped."""
    name: str = "fikizen"
    architecture: str = "fikizen"
    family: str = "fikizen"
    hidden_size: int = 256
    vocab_size: int = 512
    layers: tuple = ()
    norm_eps: float = 1e-6
    logit_softcap: float = 0.0
    max_position_embeddings: int = 1 << 20   # rotary angles are computed, not tabulated
    default_model_len: int = 32768
    bos_token_id: int | None = None
    eos_token_id: tuple = ()
    vision: object = None
    num_experts: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """Layer runs in execution order: (index of the layer that holds the weights, 0, False)."""
        return [(i if l.weights_of is None else l.weights_of, 0, False) for i, l in enumerate(self.layers)]

    def num_params(self) -> int:
        H, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size

        def mixer(m):
            if isinstance(m, WindowAttentionSpec):
                return H * (m.q_size + m.cache_dim + (m.heads if m.gate else 0)) + m.heads * m.vdim * H
            if isinstance(m, GatedDeltaSpec):
                return H * m.proj_size + m.heads * m.vdim * H
            if isinstance(m, DeltaRuleSpec):
                return 6 * H * m.size
            return mixer(m.left) + mixer(m.right)

        for l in self.layers:
            if l.weights_of is None:
                n += mixer(l.mixer) + (2 * l.mlp.ff * H if l.mlp is not None else 0)
        return n

    def replace(self, **kw) -> "FikizenConfig":
        return dataclasses.replace(self, **kw)

    @staticmethod
    def attention_spec(m: dict, **flags) -> WindowAttentionSpec:
        rot = m.get("rot") or {}
        return WindowAttentionSpec(
            heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
            scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size") or 0),
            rot_dims=int(rot.get("dims") or 0), rot_base=float(rot.get("base", 10000.0)), sink=True, **flags)

    @staticmethod
    def from_dict(d: dict, name: str = "model") -> "FikizenConfig":
        layers = []
        for l in d["layers"]:
            m, kind = l["mixer"], l["type"]
            if kind == "attention":
                mixer = FikizenConfig.attention_spec(m, gate=True)
            elif kind == "delta":
                mixer = GatedDeltaSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                       vdim=int(m["vdim"]), conv=int(m["conv"]))
            elif kind == "parallel":
                mixer = ParallelMixerSpec(
                    left=FikizenConfig.attention_spec(m["left"], bias=True, qk_norm=True, v_norm=True),
                    right=DeltaRuleSpec(heads=int(m["right"]["heads"]), dim=int(m["right"]["dim"]),
                                        decay_rank=int(m["right"].get("decay_rank") or 0)),
                    left_scale=float(m.get("left_scale", 1.0)), right_scale=float(m.get("right_scale", 1.0)))
            else:
                raise NotImplementedError(f"unknown mixer {kind!r}")
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") != "dense":
                    raise NotImplementedError(f"unknown feed-forward {f.get('kind')!r}")
                mlp = DenseFFSpec(ff=int(f["ff"]))
            wo = l.get("weights_of")
            layers.append(HybridLayerSpec(mixer, mlp, None if wo is None else int(wo)))
        for i, l in enumerate(layers):
            if l.weights_of is not None:
                j = l.weights_of
                if not (0 <= j < len(layers)) or layers[j].weights_of is not None:
                    raise ValueError(f"layer {i}: weights_of must name a layer with weights of its own")
                if (layers[j].mixer, layers[j].mlp) != (l.mixer, l.mlp):
                    raise ValueError(f"layer {i} differs from layer {j}, whose weights it uses")
        norm = d.get("norm") or {}
        eos = d.get("eos_token_id", ())
        eos = tuple(eos) if isinstance(eos, (list, tuple)) else (eos,)
        return FikizenConfig(
            name=name, hidden_size=int(d["width"]), vocab_size=int(d["vocab"]), layers=tuple(layers),
            norm_eps=float(norm.get("eps", 1e-6)), logit_softcap=float(d.get("logit_softcap") or 0.0),
            bos_token_id=d.get("bos_token_id"), eos_token_id=eos)


@dataclass(frozen=True)
class KemavikConfig:
    """Kemavik: a decoder given as a list of layers whose norms sit on the sublayers' OUTPUTS
    (``x <- x + norm(mixer(x))``, ``x <- x + norm(ff(x))``, one-plus-weight RMS norms). Mixers:
    RWKV-style linear attention with per-channel decays, or differential grouped-query
    attention with per-head query / key norms (a layer may read another layer's keys and
    values). Feed-forwards: dense with a squared ReLU, or a routed mixture of gated experts
    with identity experts and a shared expert."""
    name: str = "kemavik"
    architecture: str = "kemavik"
    family: str = "kemavik"
    hidden_size: int = 256
    vocab_size: int = 512
    layers: tuple = ()
    norm_eps: float = 1e-6
    max_position_embeddings: int = 1 << 20   # no position tables
    default_model_len: int = 32768
    bos_token_id: int | None = None
    eos_token_id: tuple = ()
    vision: object = None
    num_experts: int = 0                      # engine start-up tuning of the dense families keys on it

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """Layer runs in execution order: (layer index, 0, False); every layer runs once."""
        return [(i, 0, False) for i in range(len(self.layers))]

    def num_params(self) -> int:
        H, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        for l in self.layers:
            m, f = l.mixer, l.mlp
            if isinstance(m, WkvSpec):
                n += 5 * H * m.size + 2 * (m.decay_rank or 64) * H
            else:
                n += H * (m.q_size + m.cache_dim) + m.heads * m.vdim * H
            if isinstance(f, DenseFFSpec):
                n += 2 * f.ff * H
            elif f is not None:
                n += 3 * H * (f.experts * f.ff + f.shared_ff) + H * (f.experts + f.identity)
        return n

    def replace(self, **kw) -> "KemavikConfig":
        return dataclasses.replace(self, **kw)

    @staticmethod
    def from_dict(d: dict, name: str = "model") -> "KemavikConfig":
        layers = []
        for i, l in enumerate(d["layers"]):
            m, kind = l["mixer"], l["type"]
            if kind == "wkv":
                mixer = WkvSpec(heads=int(m["heads"]), dim=int(m["dim"]), decay_rank=int(m.get("decay_rank") or 0))
            elif kind == "attention":
                src = m.get("kv_from")
                mixer = WindowAttentionSpec(
                    heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                    scale=float(m["scale"]), bias=True, out_bias=True, head_norm=True, maps=2,
                    diff=float(m["diff"]), kv_from=None if src is None else int(src))
            else:
                raise NotImplementedError(f"unknown mixer {kind!r}")
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") == "dense":
                    mlp = DenseFFSpec(ff=int(f["ff"]), act="relu2")
                elif f.get("kind") == "moe":
                    r = f["router"]
                    mlp = RoutedMoESpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(f["expert"]["ff"]),
                                        identity=int(r.get("identity") or 0), scale=float(r.get("scale", 1.0)),
                                        shared_ff=int((f.get("shared") or {}).get("ff") or 0))
                else:
                    raise NotImplementedError(f"unknown feed-forward {f.get('kind')!r}")
            layers.append(HybridLayerSpec(mixer, mlp))
        check_kv_sources(layers)
        norm = d.get("norm") or {}
        eos = d.get("eos_token_id", ())
        eos = tuple(eos) if isinstance(eos, (list, tuple)) else (eos,)
        return KemavikConfig(
            name=name, hidden_size=int(d["width"]), vocab_size=int(d["vocab"]), layers=tuple(layers),
            norm_eps=float(norm.get("eps", 1e-6)), bos_token_id=d.get("bos_token_id"), eos_token_id=eos)


@dataclass(frozen=True)
class TopezenConfig:
    """Topezen: a decoder given as a list of layers, each a parallel block with two norms,

        x <- x + sigmoid(rg1(norm1 x)) * mixer(norm1 x) + sigmoid(rg2(norm2 x)) * ff(norm2 x)

    where the RMS norms have ONE weight each and ``rg`` are full-width projections with a bias
    (a gate per channel on each sublayer's result). Mixers: causal latent attention with an
    interleaved rotation and a per-channel output gate, an mLSTM matrix memory, or grouped-query
    attention without positions (per-head query / key norms, capped scores, a sliding window that
    keeps the first tokens, a learned softmax sink per head). Feed-forwards: dense with a
    PolyNorm activation, or a routed mixture of gated experts (corrected, group-limited top-k
    selection, renormalised weights, a shared expert); a layer may have none. The embedding is
    scaled by ``embed_scale``."""
    name: str = "topezen"
    architecture: str = "topezen"
    family: str = "topezen"
    hidden_size: int = 256
    vocab_size: int = 512
    layers: tuple = ()
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    max_position_embeddings: int = 1 << 20   # rotary angles are computed, not tabulated
    default_model_len: int = 32768
    bos_token_id: int | None = None
    eos_token_id: tuple = ()
    vision: object = None
    num_experts: int = 0                      # engine start-up tuning of the dense families keys on it

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def runs(self) -> list:
        """Layer runs in execution order: (layer index, 0, False); every layer runs once."""
        return [(i, 0, False) for i in range(len(self.layers))]

    def num_params(self) -> int:
        H, n = self.hidden_size, 2 * self.vocab_size * self.hidden_size
        for l in self.layers:
            m, f = l.mixer, l.mlp
            n += H * H
            if isinstance(m, LatentAttentionSpec):
                n += H * (m.q_rank + m.key_dim + m.gate_size) + m.q_rank * m.heads * (m.dim + m.rot_dim)
                n += m.kv_rank * m.heads * (m.dim + m.vdim) + m.heads * m.vdim * H
            elif isinstance(m, MLstmSpec):
                n += H * (2 * m.heads * m.dim + 3 * m.out_size + 2 * m.heads)
            else:
                n += H * (m.q_size + m.cache_dim) + m.heads * m.vdim * H
            if f is not None:
                n += H * H
            if isinstance(f, DenseFFSpec):
                n += 2 * f.ff * H
            elif f is not None:
                n += 3 * H * (f.experts * f.ff + f.shared_ff) + H * f.experts
        return n

    def replace(self, **kw) -> "TopezenConfig":
        return dataclasses.replace(self, **kw)

    @staticmethod
    def from_dict(d: dict, name: str = "model") -> "TopezenConfig":
        layers = []
        for l in d["layers"]:
            m, kind = l["mixer"], l["type"]
            if kind == "latent_attention":
                rot = m.get("rot") or {}
                mixer = LatentAttentionSpec(
                    heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                    q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                    rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims") or m["rot_dim"]),
                    interleaved=True, gate="channel")
            elif kind == "mlstm":
                mixer = MLstmSpec(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                                  gate_cap=float(m["gate_cap"]))
            elif kind == "attention":
                mask = m.get("mask") or {}
                mixer = WindowAttentionSpec(
                    heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                    scale=float(m["scale"]), window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0),
                    softcap=float(m.get("softcap") or 0.0), head_norm=True, sink=True, sink_weights=True)
            else:
                raise NotImplementedError(f"unknown mixer {kind!r}")
            f = l.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind") == "dense":
                    mlp = DenseFFSpec(ff=int(f["ff"]), act="polynorm")
                elif f.get("kind") == "moe":
                    r = f["router"]
                    g = r.get("groups") or {}
                    count = int(g.get("count") or 1)
                    if int(r["experts"]) % count:
                        raise ValueError("the experts do not divide into equal groups")
                    mlp = RoutedMoESpec(experts=int(r["experts"]), top=int(r["top"]), ff=int(f["expert"]["ff"]),
                                        shared_ff=int((f.get("shared") or {}).get("ff") or 0), groups=count,
                                        keep_groups=int(g.get("keep") or count), renorm=True)
                else:
                    raise NotImplementedError(f"unknown feed-forward {f.get('kind')!r}")
            layers.append(HybridLayerSpec(mixer, mlp))
        norm = d.get("norm") or {}
        eos = d.get("eos_token_id", ())
        eos = tuple(eos) if isinstance(eos, (list, tuple)) else (eos,)
        return TopezenConfig(
            name=name, hidden_size=int(d["width"]), vocab_size=int(d["vocab"]), layers=tuple(layers),
            norm_eps=float(norm.get("eps", 1e-6)), embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
            bos_token_id=d.get("bos_token_id"), eos_token_id=eos)


def check_kv_sources(layers):
    """A layer that reads another layer's keys and values must name an earlier attention layer
    with a cache of its own and the same key / value head layout."""
    for i, l in enumerate(layers):
        j = getattr(l.mixer, "kv_from", None)
        if j is None:
            continue
        if not (0 <= j < i) or not isinstance(layers[j].mixer, WindowAttentionSpec) or layers[j].mixer.kv_from is not None:
            raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys and values of its own")
        a, b = l.mixer, layers[j].mixer
        if (a.kv_heads, a.maps, a.dim, a.vdim) != (b.kv_heads, b.maps, b.dim, b.vdim):
            raise ValueError(f"layer {i}: its key / value heads differ from those of layer {j}, whose cache it reads")


def config_from_dict(d: dict, name: str = "model"):
    """Model config of a ``config.json``: the layer-list designs are recognised by their
    ``architecture`` key, everything else is a HuggingFace config."""
    arch = str(d.get("architecture", "")).lower()
    if arch == "kesirax":
        return HybridConfig.from_dict(d, name=name)
    if arch == "fikizen":
        return FikizenConfig.from_dict(d, name=name)
    if arch == "kemavik":
        return KemavikConfig.from_dict(d, name=name)
    if arch == "topezen":
        return TopezenConfig.from_dict(d, name=name)
    return ModelConfig.from_hf_dict(d, name=name)


def _mini_kesirax(name, H, V, attn, gru, ff, order, loop=(0, 0, 1), groups=1):
    a = LatentAttentionSpec(**attn)
    g = MinGRUSpec(gru)
    f = TableMoESpec(**ff) if ff else None
    return HybridConfig(name=name, hidden_size=H, vocab_size=V,
                        layers=tuple(HybridLayerSpec(a if c == "a" else g, f) for c in order),
                        loop_start=loop[0], loop_stop=loop[1], loop_times=loop[2], norm_groups=groups,
                        eos_token_id=(2,), bos_token_id=1)


PRESETS.update({
    # CPU plumbing size
    "tiny-kesirax": _mini_kesirax("tiny-kesirax", 64, 320,
                                  dict(heads=3, dim=16, rot_dim=8, vdim=24, q_rank=40, kv_rank=32, scale=24 ** -0.5,
                                       window=24, rot_base=10000.0),
                                  48, dict(experts=4, top=2, ff=40), "agga", loop=(1, 3, 2), groups=4),
    # GPU-test size
    "small-kesirax": _mini_kesirax("small-kesirax", 512, 1024,
                                   dict(heads=8, dim=64, rot_dim=32, vdim=64, q_rank=192, kv_rank=128,
                                        scale=96 ** -0.5, window=160, rot_base=50000.0),
                                   768, dict(experts=8, top=2, ff=256), "agag", loop=(0, 2, 2), groups=2),
})


def _mini_fikizen(name, H, V, attn, left, delta, rule, ff, order, scales=(0.75, 1.25), softcap=20.0):
    """order: 'd' gated delta rule (no feed-forward), 'a' gated sink attention + feed-forward, 'p' parallel
    mixer + feed-forward, 'A' the first 'a' layer's weights once more."""
    a = WindowAttentionSpec(sink=True, gate=True, **attn)
    p = ParallelMixerSpec(WindowAttentionSpec(sink=True, bias=True, qk_norm=True, v_norm=True, **left),
                          DeltaRuleSpec(**rule), *scales)
    f = DenseFFSpec(ff)
    first = order.index("a") if "A" in order else None
    spec = {"d": HybridLayerSpec(GatedDeltaSpec(**delta), None), "a": HybridLayerSpec(a, f),
            "p": HybridLayerSpec(p, f), "A": HybridLayerSpec(a, f, first)}
    return FikizenConfig(name=name, hidden_size=H, vocab_size=V, layers=tuple(spec[c] for c in order),
                         logit_softcap=softcap, eos_token_id=(2,), bos_token_id=1)


PRESETS.update({
    # CPU plumbing size
    "tiny-fikizen": _mini_fikizen("tiny-fikizen", 64, 320,
                                  dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.25, window=24, rot_dims=8),
                                  dict(heads=3, kv_heads=3, dim=16, vdim=16, scale=0.25, window=16, rot_dims=16),
                                  dict(heads=4, kv_heads=2, dim=8, vdim=12, conv=3), dict(heads=2, dim=16, decay_rank=8),
                                  96, "apdAd"),
    # GPU-test size
    "small-fikizen": _mini_fikizen("small-fikizen", 512, 1024,
                                   dict(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.125, window=160, rot_dims=32,
                                        rot_base=5e5),
                                   dict(heads=8, kv_heads=4, dim=64, vdim=64, scale=0.125, window=80, rot_dims=64),
                                   dict(heads=8, kv_heads=4, dim=64, vdim=64, conv=3), dict(heads=8, dim=64, decay_rank=32),
                                   1536, "adAp"),
})


def _mini_kemavik(name, H, V, wkv, attn, ff, moe, order):
    """order: 'w' linear attention + dense feed-forward, 'a' differential attention + routed experts,
    's' differential attention on the keys and values of the nearest 'a' before it + dense feed-forward,
    'n' linear attention without a feed-forward."""
    layers = []
    for c in order:
        if c in "wn":
            layers.append(HybridLayerSpec(WkvSpec(**wkv), DenseFFSpec(ff, "relu2") if c == "w" else None))
        else:
            src = max(i for i, o in enumerate(order[:len(layers)]) if o == "a") if c == "s" else None
            a = WindowAttentionSpec(bias=True, out_bias=True, head_norm=True, maps=2, kv_from=src, **attn)
            layers.append(HybridLayerSpec(a, RoutedMoESpec(**moe) if c == "a" else DenseFFSpec(ff, "relu2")))
    return KemavikConfig(name=name, hidden_size=H, vocab_size=V, layers=tuple(layers), eos_token_id=(2,),
                         bos_token_id=1)


PRESETS.update({
    # CPU plumbing size
    "tiny-kemavik": _mini_kemavik("tiny-kemavik", 64, 320, dict(heads=2, dim=16, decay_rank=8),
                                  dict(heads=4, kv_heads=2, dim=8, vdim=24, scale=0.3, diff=0.4), 96,
                                  dict(experts=5, top=2, ff=24, identity=2, scale=1.5, shared_ff=40), "wasaw"),
    # GPU-test size
    "small-kemavik": _mini_kemavik("small-kemavik", 512, 1024, dict(heads=8, dim=64, decay_rank=32),
                                   dict(heads=8, kv_heads=2, dim=32, vdim=64, scale=32 ** -0.5, diff=0.5), 1536,
                                   dict(experts=8, top=2, ff=256, identity=2, scale=1.0, shared_ff=512), "wasw"),
})


def _mini_topezen(name, H, V, latent, mlstm, attn, ff, moe, order, embed_scale=4.0):
    """order: 'l' latent attention + dense feed-forward, 'm' matrix memory + routed experts, 'a' capped window
    attention with a learned sink + routed experts, 'n' matrix memory without a feed-forward."""
    f, e = DenseFFSpec(ff, "polynorm"), RoutedMoESpec(renorm=True, **moe)
    spec = {"l": HybridLayerSpec(LatentAttentionSpec(interleaved=True, gate="channel", **latent), f),
            "m": HybridLayerSpec(MLstmSpec(**mlstm), e),
            "a": HybridLayerSpec(WindowAttentionSpec(head_norm=True, sink=True, sink_weights=True, **attn), e),
            "n": HybridLayerSpec(MLstmSpec(**mlstm), None)}
    return TopezenConfig(name=name, hidden_size=H, vocab_size=V, layers=tuple(spec[c] for c in order),
                         embed_scale=embed_scale, eos_token_id=(2,), bos_token_id=1)


PRESETS.update({
    # CPU plumbing size
    "tiny-topezen": _mini_topezen("tiny-topezen", 64, 320,
                                  dict(heads=3, dim=16, rot_dim=8, vdim=24, q_rank=40, kv_rank=32, scale=24 ** -0.5),
                                  dict(heads=2, dim=16, vdim=24, gate_cap=10.0),
                                  dict(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.25, window=24, keep_first=5, softcap=30.0),
                                  96, dict(experts=6, top=2, ff=24, shared_ff=40, groups=3, keep_groups=2), "lmanl"),
    # GPU-test size
    "small-topezen": _mini_topezen("small-topezen", 512, 1024,
                                   dict(heads=8, dim=64, rot_dim=32, vdim=64, q_rank=192, kv_rank=128, scale=96 ** -0.5,
                                        rot_base=50000.0),
                                   dict(heads=4, dim=64, vdim=128, gate_cap=15.0),
                                   dict(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.125, window=160, keep_first=16,
                                        softcap=50.0),
                                   1536, dict(experts=8, top=2, ff=256, shared_ff=512, groups=4, keep_groups=2), "lmam"),
})
