"""What the layer-list decoders share: weight holders per layer that owns weights, checkpoint
loading by the designs' tensor names, random checkpoints, and the paged cache / state tensors
per layer RUN. A design subclasses ``LayerListModel`` and writes its ``forward`` (how mixer,
feed-forward, norms and the residual stream are composed) and ``compute_logits``.

Layer options the base class understands (``config.HybridLayerSpec`` and the mixer specs):
``weights_of`` (a layer runs another layer's weights, with a cache / state of its own) and a
mixer's ``kv_from`` (an attention layer reads another layer run's paged cache instead of
having one).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ..parallel.comm import TPGroup
from .mixers import make_ff, make_mixer


class _Layer:
    def __init__(self):
        self.norm1 = self.norm2 = None   # [hidden] fp32 (one number each in designs with single-weight norms)
        self.b1 = self.b2 = None         # [hidden] fp32: biases of the gates on the sublayers' results, where a design has them
        self.mixer = None
        self.mlp = None


class LayerListModel:
    supports_fp32 = True        # every op of these models has a true 32-bit build
    graph_decode = True         # decode-only steps replay a captured hipGraph
    norm_offset = 0.0           # added to every norm weight at load (1.0: weights stored around zero)
    norm_library = "delta"      # the kernel library whose residual + norm kernels run (the one the mixers load)

    def __init__(self, cfg, tp: TPGroup, device, dtype=torch.bfloat16, ops=None, max_pos: int | None = None):
        if tp.world_size != 1:
            raise NotImplementedError("the layer-list decoders run on one device (TP = 1)")
        self.cfg, self.tp, self.ops = cfg, tp, ops
        if hasattr(ops, "norm_library"):
            ops.norm_library = self.norm_library
        self.device, self.dtype = torch.device(device), dtype
        self.kv_dtype = dtype
        self.vpad = cfg.vocab_size
        self.visual = None
        self.decode_partition = 512
        self.block_size_hint = 16
        self.runs = cfg.runs()
        # weight holders only for the layers that own weights
        self.layers: list[_Layer | None] = []
        H = cfg.hidden_size
        for spec in cfg.layers:
            if spec.weights_of is not None:
                self.layers.append(None)
                continue
            lw = _Layer()
            lw.mixer = make_mixer(spec.mixer, H, cfg.norm_eps, self.device, dtype, ops)
            if spec.mlp is not None:
                lw.mlp = make_ff(spec.mlp, H, self.device, dtype, ops, cfg.norm_eps)
            self.layers.append(lw)
        self.embed = self.final_norm = self.lm_head = None
        self.capture = None  # a list: the residual stream after every layer run is appended (debugging)

    # ---------------------------------------------------------------- weights
    @property
    def needs_state(self) -> bool:
        return any(self.layers[i].mixer.state_shapes for i, _, _ in self.runs)

    def load_tensors(self, get):
        """``get(name)`` -> CPU tensor of the checkpoint (names: ``embed``, ``head``, ``final.norm``,
        ``l<i>.norm1`` / ``.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*`` for the layers with weights of their own)."""
        dev, dt = self.device, self.dtype
        self.embed = get("embed").to(dev, dt).contiguous()
        self.lm_head = get("head").to(dev, dt).contiguous()
        self.final_norm = get("final.norm").to(dev, torch.float32) + self.norm_offset
        for i, lw in enumerate(self.layers):
            if lw is None:
                continue
            lw.norm1 = get(f"l{i}.norm1").to(dev, torch.float32) + self.norm_offset
            lw.mixer.load(get, f"l{i}.mix.")
            if lw.mlp is not None:
                lw.norm2 = get(f"l{i}.norm2").to(dev, torch.float32) + self.norm_offset
                lw.mlp.load(get, f"l{i}.mlp.")

    def random_tensors(self, seed: int = 0, std: float = 0.05) -> dict:
        """Random checkpoint tensors (bf16-representable values) under the checkpoint's names."""
        cfg = self.cfg
        g = torch.Generator().manual_seed(seed)
        H, V = cfg.hidden_size, cfg.vocab_size
        out = {"embed": torch.randn(V, H, generator=g), "head": torch.randn(V, H, generator=g) * std * 4,
               "final.norm": 1.0 - self.norm_offset + 0.1 * torch.randn(H, generator=g)}
        for i, lw in enumerate(self.layers):
            if lw is None:
                continue
            out[f"l{i}.norm1"] = 1.0 - self.norm_offset + 0.1 * torch.randn(H, generator=g)
            for k, v in lw.mixer.init_random(g, std).items():
                out[f"l{i}.mix.{k}"] = v
            if lw.mlp is not None:
                out[f"l{i}.norm2"] = 1.0 - self.norm_offset + 0.1 * torch.randn(H, generator=g)
                for k, v in lw.mlp.init_random(g, std).items():
                    out[f"l{i}.mlp.{k}"] = v
        return {k: v.bfloat16().float() for k, v in out.items()}

    def allocate_random(self, seed: int = 0, std: float = 0.05):
        t = self.random_tensors(seed, std)
        self.load_tensors(lambda k: t[k])

    def allocate_random_quant(self, scheme: str, seed: int = 0):
        raise NotImplementedError("quantised weights are not available for this architecture")

    # ---------------------------------------------------------------- cache / state
    def _mixer(self, r: int):
        return self.layers[self.runs[r][0]].mixer

    def kv_bytes_per_block(self, block_size: int) -> int:
        el = torch.finfo(self.kv_dtype).bits // 8
        return max(1, sum(self._mixer(r).cache_dim for r in range(len(self.runs))) * block_size * el)

    def allocate_kv_cache(self, num_blocks: int, block_size: int):
        """One paged cache per layer RUN with attention: [num_blocks, block_size, all key heads | all value
        heads]; all runs share the sequences' block tables. A run whose mixer names another layer's keys and
        values (``kv_from``) gets that run's tensor."""
        kv = [None] * len(self.runs)
        for r in range(len(self.runs)):
            n = self._mixer(r).cache_dim
            if n:
                kv[r] = torch.zeros(num_blocks, block_size, n, device=self.device, dtype=self.kv_dtype)
        for r in range(len(self.runs)):
            src = getattr(getattr(self._mixer(r), "spec", None), "kv_from", None)
            if src is not None:
                kv[r] = kv[src]
        return kv

    def state_bytes_per_slot(self) -> int:
        n = 0
        for r in range(len(self.runs)):
            f = self._mixer(r).state_shapes
            for shape in (f(1) if f else []):
                n += 4 * int(torch.tensor(shape).prod())
        return n

    def allocate_state(self, num_slots: int):
        """32-bit state tensors per layer run with a recurrence, indexed by sequence slot."""
        st = [None] * len(self.runs)
        for r in range(len(self.runs)):
            f = self._mixer(r).state_shapes
            if f:
                st[r] = [torch.zeros(shape, device=self.device, dtype=torch.float32) for shape in f(num_slots)]
        return st

    def step_workspace_bytes(self, tokens: int, seqs: int) -> int:
        el = torch.finfo(self.dtype).bits // 8
        wide = 0
        for lw in self.layers:
            if lw is None:
                continue
            n = 3 * _proj_width(lw.mixer)
            if lw.mlp is not None:
                f = lw.mlp.spec
                n = max(n, 2 * f.ff * getattr(f, "top", 1) * 2 + 2 * getattr(f, "shared_ff", 0))
            wide = max(wide, n)
        return tokens * (wide * (el + 4) + 12 * self.cfg.hidden_size) + seqs * self.cfg.vocab_size * 12

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """32-bit logits = head . hidden."""
        if hidden.dtype == torch.float32:
            return F.linear(hidden, self.lm_head)
        if hidden.is_cuda:
            return torch.mm(hidden, self.lm_head.t(), out_dtype=torch.float32)
        return F.linear(hidden.float(), self.lm_head.float())


def _proj_width(mixer) -> int:
    """Columns of a mixer's input projections (all of them together)."""
    if hasattr(mixer, "left"):
        return _proj_width(mixer.left) + _proj_width(mixer.right)
    if hasattr(mixer, "w_in_t"):   # batched projections [n, hidden, out] of n blended copies of the input
        return mixer.w_in_t.shape[0] * mixer.w_in_t.shape[2] + (mixer.w_in_t.shape[0] + 1) * mixer.hidden
    return mixer.w_in.shape[0]
