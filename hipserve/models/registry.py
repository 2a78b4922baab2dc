"""Model registry: which model class serves a model config. The engine (model runner,
weight loading, CLI) goes through ``build_model`` / ``load_weights`` and never names a
model class itself.

A registered class is constructed as ``cls(cfg, tp, device, dtype, ops, max_pos=...)`` and
offers ``forward(ids, meta, kv)``, ``compute_logits(hidden)``, ``allocate_kv_cache`` /
``kv_bytes_per_block``, ``allocate_random`` and the attributes ``vpad`` / ``visual``.
Optional capabilities the runner asks for by attribute:

* ``supports_fp32``  the model's kernels have a true 32-bit build (``--dtype float32`` on a GPU)
* ``needs_state`` + ``allocate_state(slots)``  per-sequence recurrent state slots
* ``graph_decode = False``  decode steps are not captured into hipGraphs
* ``gemm_shapes`` etc.  the dense-transformer start-up tuning (decode GEMM autotune, packing)
"""
from __future__ import annotations

import importlib

# architecture (``config.architecture``) -> (module, class, weight loader "module:function")
ARCHITECTURES = {
    "llama": ("hipserve.models.llama", "LlamaModel", "hipserve.weights.safetensors_loader:load_hf_weights"),
    "mixtral": ("hipserve.models.llama", "LlamaModel", "hipserve.weights.safetensors_loader:load_hf_weights"),
    "kesirax": ("hipserve.models.kesirax", "KesiraxModel", "hipserve.weights.safetensors_loader:load_named_tensors"),
    "fikizen": ("hipserve.models.fikizen", "FikizenModel", "hipserve.weights.safetensors_loader:load_named_tensors"),
    "kemavik": ("hipserve.models.kemavik", "KemavikModel", "hipserve.weights.safetensors_loader:load_named_tensors"),
    "topezen": ("hipserve.models.topezen", "TopezenModel", "hipserve.weights.safetensors_loader:load_named_tensors"),
}


def model_class(mcfg):
    try:
        mod, cls, _ = ARCHITECTURES[mcfg.architecture]
    except KeyError:
        raise NotImplementedError(f"no model class for architecture {mcfg.architecture!r}") from None
    return getattr(importlib.import_module(mod), cls)


def build_model(mcfg, tp, device, dtype, ops, max_pos=None):
    return model_class(mcfg)(mcfg, tp, device, dtype, ops, max_pos=max_pos)


def load_weights(model, path: str):
    """Load a safetensors checkpoint into ``model`` with its architecture's loader."""
    mod, fn = ARCHITECTURES[model.cfg.architecture][2].split(":")
    return getattr(importlib.import_module(mod), fn)(model, path)
