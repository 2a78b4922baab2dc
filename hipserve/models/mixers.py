"""Sequence mixers and feed-forwards of the layer-list decoders, as weight holders with a
``forward`` over the flat token rows of one engine step. Each is parameterised by its
spec (``config.LatentAttentionSpec`` / ``MinGRUSpec`` / ``TableMoESpec``) and runs on the
engine's op set (``ops.KernelOps`` on a GPU, ``ops.ReferenceOps`` on the CPU), so another
design can list them in its own layer order.

Dense projections are vendor GEMMs (``F.linear`` / ``torch.bmm``); everything between
them is one op of the op set:

* latent attention: merged [q-latent | kv-latent | rotary key | gate] projection ->
  ``latent_prepare`` (both latent RMSNorms, rotary key part, paged cache write) -> query
  up-projection -> per-head absorption of the key up-projection into the query (so the
  attention runs directly on the cached latents, one shared "key head" for all heads) ->
  ``latent_attention`` (rotary query part, sliding window, softmax, output gate) ->
  per-head value up-projection -> output projection.
* minGRU: merged [z | x | g] projection -> ``mingru_scan`` (gates, candidate, the
  recurrence over this step's tokens from the sequence's state slot, output gate) ->
  output projection.
* table MoE: expert ids looked up by token id -> ``moe_align`` tiles -> two
  ``expert_gemm`` launches (squared-ReLU in the first one's epilogue); the weighted
  combine is folded into the residual update (``scaled_add_group_rmsnorm``).
* window attention: merged [q | k | v | gate] projection (biases in its epilogue) ->
  ``attn_prepare`` (whole-projection or per-head q / k norm, rotation, value norm, paged cache
  write) -> ``window_attention`` (sliding window, softmax with a sink, per-head output gate; with
  two maps per head the differential combination and its norm) -> output projection. A layer
  that reads another layer's cache projects only its queries.
* linear attention with per-channel decays (``Wkv``): ``token_shift`` (five blends of the token's
  and the previous token's 32-bit input) -> one batched projection for r / k / v / gate and the
  decay bottleneck -> tanh -> decay up-projection (32-bit result) -> ``wkv`` (decay, bonus, the
  recurrence from the sequence's state slot, per-head output norm and SiLU gate) -> output
  projection.
* routed experts (``RoutedMoE``): 32-bit router logits -> ``route_topk`` (softmax, corrected
  selection, weights) -> ``moe_align`` tiles -> ``expert_gemm`` (gate | up, SiLU gate in its epilogue)
  -> ``expert_gemm`` (down); the weighted combine, the identity experts and the shared
  expert are folded into the residual update (``add_normed``).
* gated delta rule: merged [q | k | v | beta | decay | gate] projection -> ``gated_delta``
  (causal convolution + SiLU, unit q / k, the recurrence from the sequence's state slot,
  per-head output norm and SiLU gate) -> output projection.
* generalized delta rule: merged [r | k | v | a | g | decay bottleneck] projection -> tanh ->
  decay up-projection (32-bit result) -> ``delta_rule`` (decay, removal rate, unit key, the
  recurrence, per-head output norm and sigmoid gate) -> output projection.
* parallel mixer: both halves write their scaled head outputs side by side into one
  buffer, and ONE output projection over the concatenated weights sums them.
* dense feed-forward: up projection -> ``activation`` -> down projection.

* matrix memory (``MLstm``): merged [q | k | v | gate] projection and a 32-bit [input gate | forget
  gate] projection -> ``mlstm`` (capped log gates, running maximum, the recurrence of the matrix
  state and its normaliser from the sequence's state slot, read-out, per-head output norm, weight
  and sigmoid gate) -> output projection.

A mixer's ``forward(h, meta, cache, state)`` gets the layer run's paged cache and state
tensors (None where it has none); ``cache_dim`` / ``state_shapes`` say what a run needs.

Side projection: a model whose block needs one more projection of a sublayer's input (a gate on
the sublayer's result, say) attaches its rows to the sublayer's merged input GEMM with
``attach_side``; after ``forward`` the sublayer's ``side_out`` holds those columns.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ..config import (DeltaRuleSpec, DenseFFSpec, GatedDeltaSpec, LatentAttentionSpec, MinGRUSpec, MLstmSpec,
                      ParallelMixerSpec, RoutedMoESpec, TableMoESpec, WindowAttentionSpec, WkvSpec)

MOE_TILE = 32        # slots per expert tile of the expert GEMMs ...
MOE_TILE_LARGE = 64  # ... when every expert has several tiles' worth of rows on average
# bf16 batches with at least this many (token, expert) pairs per expert run the packed-layout grouped
# GEMM of the dense families' MoE prefill (prefill_gemm_packed.hip: 128-row tiles, X through LDS, the
# weights pre-shuffled into MFMA operand order) with the squared ReLU in its epilogue
MOE_PACKED_MIN_PAIRS_PER_EXPERT = 256


def attach_side(sub, w: torch.Tensor):
    """Append the rows of ``w`` [n, hidden] to the merged input projection of a mixer or feed-forward."""
    name = sub.side_weight
    cur = getattr(sub, name)
    w = w.to(sub.device, sub.dtype)
    setattr(sub, name, w.contiguous() if cur is None else torch.cat([cur, w], 0).contiguous())
    if getattr(sub, "b_in", None) is not None:
        sub.b_in = torch.cat([sub.b_in, torch.zeros(w.shape[0], device=sub.device, dtype=sub.b_in.dtype)]).contiguous()
    sub.side_rows = w.shape[0]


def _side(sub, proj: torch.Tensor):
    n = sub.side_rows
    sub.side_out = proj[:, proj.shape[1] - n:] if n else None


def _deinterleave(w: torch.Tensor, dims: int) -> torch.Tensor:
    """Rows [..., r, in] of a projection whose outputs are rotated in pairs (2i, 2i + 1): the first ``dims`` rows
    reordered to [even | odd], so that the rotate-half kernels (pairs i, i + dims / 2) compute the same scores."""
    idx = torch.cat([torch.arange(0, dims, 2), torch.arange(1, dims, 2), torch.arange(dims, w.shape[-2])])
    return w.index_select(-2, idx)


def _mm32(x: torch.Tensor, w_t: torch.Tensor) -> torch.Tensor:
    """Batched product with a 32-bit result (the attention's query side stays 32-bit)."""
    if x.dtype == torch.float32:
        return torch.bmm(x, w_t)
    if x.is_cuda:
        return torch.bmm(x, w_t, out_dtype=torch.float32)
    return torch.bmm(x.float(), w_t.float())


class LatentAttention:
    side_weight, side_rows, side_out = "w_in", 0, None
    state_shapes = None
    cache_dim = property(lambda self: self.spec.key_dim)

    def __init__(self, spec: LatentAttentionSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.eps, self.device, self.dtype, self.ops = spec, hidden, eps, device, dtype, ops
        s = spec
        assert s.gate in ("head", "channel", "none")
        self.w_in = None       # [q_rank + kv_rank + rot_dim + gate rows, hidden]
        self.q_norm = None     # [q_rank] fp32
        self.kv_norm = None    # [kv_rank] fp32
        self.w_uq = None       # [heads * (dim + rot_dim), q_rank]
        self.w_uk = None       # [heads, dim, kv_rank]
        self.w_uk_wide = None  # [heads, dim, kv_rank + rot_dim], zero rotary columns (made at first use)
        self.w_uv_t = None     # [heads, kv_rank, vdim]
        self.w_o = None        # [hidden, heads * vdim]
        rd = s.rot_dims or s.rot_dim
        i = torch.arange(rd // 2, dtype=torch.float32)
        # f_i = base^(-2i / dims), 32-bit
        self.inv_freq = torch.pow(torch.tensor(s.rot_base, dtype=torch.float32), -2.0 * i / rd).to(device)

    def load(self, get, prefix: str):
        s, dt, dev = self.spec, self.dtype, self.device
        dkv, uq = get(prefix + "dkv"), get(prefix + "uq")
        if s.interleaved:
            # the same permutation of the rotary key rows and of every head's rotary query rows leaves the
            # scores unchanged and turns the pairs (2i, 2i + 1) into the pairs (i, i + dims / 2) of the kernels
            rd = s.rot_dims or s.rot_dim
            dkv = torch.cat([dkv[: s.kv_rank], _deinterleave(dkv[s.kv_rank:], rd)], 0)
            uq = uq.view(s.heads, s.dim + s.rot_dim, -1)
            uq = torch.cat([uq[:, : s.dim], _deinterleave(uq[:, s.dim:], rd)], 1).reshape(-1, uq.shape[-1])
        parts = [get(prefix + "dq"), dkv] + ([get(prefix + "g")] if s.gate != "none" else [])
        self.w_in = torch.cat(parts, 0).to(dev, dt).contiguous()
        self.q_norm = get(prefix + "dq.norm").to(dev, torch.float32)
        self.kv_norm = get(prefix + "dkv.norm").to(dev, torch.float32)
        self.w_uq = uq.to(dev, dt).contiguous()
        self.w_uk = get(prefix + "uk").to(dev, dt).view(s.heads, s.dim, s.kv_rank).contiguous()
        self.w_uv_t = get(prefix + "uv").to(dev, dt).view(s.heads, s.vdim, s.kv_rank).transpose(1, 2).contiguous()
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden

        def w(*shape, scale=1.0):
            return torch.randn(*shape, generator=gen) * std * scale

        t = {"dq": w(s.q_rank, H), "dkv": w(s.key_dim, H), "g": w(max(s.gate_size, 1), H, scale=4.0 if s.gate == "channel" else 1.0),
             "dq.norm": 1.0 + 0.1 * torch.randn(s.q_rank, generator=gen),
             "dkv.norm": 1.0 + 0.1 * torch.randn(s.kv_rank, generator=gen),
             "uq": w(s.heads * (s.dim + s.rot_dim), s.q_rank, scale=4.0), "uk": w(s.heads * s.dim, s.kv_rank, scale=4.0),
             "uv": w(s.heads * s.vdim, s.kv_rank, scale=4.0), "o": w(H, s.heads * s.vdim)}
        if s.gate == "none":
            del t["g"]
        self.load(lambda k: t[k], "")
        return t

    def cache_shape(self, num_blocks: int, block_size: int):
        return (num_blocks, block_size, self.spec.key_dim)

    def forward(self, h: torch.Tensor, meta, cache: torch.Tensor, state=None) -> torch.Tensor:
        s, ops = self.spec, self.ops
        T = h.shape[0]
        proj = F.linear(h, self.w_in)
        _side(self, proj)
        gate_off = s.q_rank + s.key_dim
        cq = torch.empty(T, s.q_rank, device=h.device, dtype=h.dtype)
        ops.latent_prepare(cq, cache, proj, meta.positions, meta.slot_mapping, self.q_norm, self.kv_norm,
                           self.inv_freq, s.q_rank, s.kv_rank, s.rot_dim, self.eps)
        q = F.linear(cq, self.w_uq)                                    # [T, heads * (dim + rot_dim)]
        qh = q.view(T, s.heads, s.dim + s.rot_dim)
        if ops.latent_query_in_place(h.dtype, s.kv_rank, s.rot_dim):
            # the absorption GEMM writes the attention kernel's query rows directly: bf16, the cached width,
            # zero weight columns where the attention op puts the rotated part
            if self.w_uk_wide is None:
                self.w_uk_wide = F.pad(self.w_uk, (0, s.rot_dim)).contiguous()
            q_abs = torch.bmm(qh[:, :, : s.dim].transpose(0, 1), self.w_uk_wide)   # [heads, T, kv_rank + rot_dim]
        else:
            q_abs = _mm32(qh[:, :, : s.dim].transpose(0, 1), self.w_uk)            # [heads, T, kv_rank] fp32
        o_lat = torch.empty(s.heads, T, s.kv_rank, device=h.device, dtype=h.dtype)
        ops.latent_attention(o_lat, q_abs, q, proj, cache, meta, self.inv_freq, s.heads, s.dim, s.rot_dim,
                             s.kv_rank, gate_off if s.gate == "head" else -1, s.scale, s.window)
        o = torch.bmm(o_lat, self.w_uv_t)                              # [heads, T, vdim]
        if s.gate == "channel":
            # heads side by side per token, each element times the sigmoid of its gate column: one pass
            cat = torch.empty(T, s.heads * s.vdim, device=h.device, dtype=h.dtype)
            ops.gate_mul(cat, o, proj[:, gate_off:gate_off + s.heads * s.vdim])
            return F.linear(cat, self.w_o)
        return F.linear(o.transpose(0, 1).reshape(T, s.heads * s.vdim), self.w_o)


class MinGRU:
    def __init__(self, spec: MinGRUSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.device, self.dtype, self.ops = spec, hidden, device, dtype, ops
        self.w_in = None   # [3 * width, hidden]: z | x | g
        self.b_z = None    # [width] fp32
        self.b_x = None
        self.w_o = None    # [hidden, width]

    def load(self, get, prefix: str):
        dt, dev = self.dtype, self.device
        self.w_in = torch.cat([get(prefix + "z"), get(prefix + "x"), get(prefix + "g")], 0).to(dev, dt).contiguous()
        self.b_z = get(prefix + "z.b").to(dev, torch.float32)
        self.b_x = get(prefix + "x.b").to(dev, torch.float32)
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        n, H = self.spec.width, self.hidden
        t = {k: torch.randn(n, H, generator=gen) * std * 4.0 for k in ("z", "x", "g")}
        t["z.b"] = torch.randn(n, generator=gen)
        t["x.b"] = torch.randn(n, generator=gen) * 0.5
        t["o"] = torch.randn(H, n, generator=gen) * std
        self.load(lambda k: t[k], "")
        return t

    def state_shape(self, num_slots: int):
        return (num_slots, self.spec.width)

    def forward(self, h: torch.Tensor, meta, state: torch.Tensor) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        y = torch.empty(h.shape[0], self.spec.width, device=h.device, dtype=h.dtype)
        self.ops.mingru_scan(y, state, proj, self.b_z, self.b_x, meta)
        return F.linear(y, self.w_o)


class TableMoE:
    """``forward`` returns (y [slots, hidden], pair_slot [T * top]): row ``pair_slot[t * top + j]``
    of ``y`` is token t's j-th expert output; the caller sums them with weight 1 / top."""

    def __init__(self, spec: TableMoESpec, hidden: int, vocab: int, device, dtype, ops):
        self.spec, self.hidden, self.vocab, self.device, self.dtype, self.ops = spec, hidden, vocab, device, dtype, ops
        self.table = None   # int32 [vocab, top]
        self.w_up = None    # [E, ff, hidden]
        self.w_down = None  # [E, hidden, ff]
        self.packed = None  # (up, down) in the packed grouped-GEMM layout, made at the first large batch

    def load(self, get, prefix: str):
        dt, dev, E = self.dtype, self.device, self.spec.experts
        self.table = get(prefix + "table").to(dev, torch.int32).contiguous()
        self.w_up = torch.stack([get(f"{prefix}e{e}.up") for e in range(E)]).to(dev, dt).contiguous()
        self.w_down = torch.stack([get(f"{prefix}e{e}.down") for e in range(E)]).to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden
        t = {"table": torch.stack([torch.randperm(s.experts, generator=gen)[: s.top] for _ in range(self.vocab)]).int()}
        for e in range(s.experts):
            t[f"e{e}.up"] = torch.randn(s.ff, H, generator=gen) * std * 4.0
            t[f"e{e}.down"] = torch.randn(H, s.ff, generator=gen) * std * 4.0
        self.load(lambda k: t[k], "")
        return t

    def forward(self, h: torch.Tensor, ids: torch.Tensor):
        s, ops = self.spec, self.ops
        T, dev = h.shape[0], h.device
        experts = self.table.index_select(0, ids).reshape(-1)          # [T * top]
        P = T * s.top
        if self._packed_ok(h, P):
            return self._forward_packed(h, experts, P)
        tile = MOE_TILE_LARGE if P >= 4 * MOE_TILE_LARGE * s.experts else MOE_TILE
        cap = -(-(P + s.experts * (tile - 1)) // tile) * tile
        slots = torch.empty(cap, dtype=torch.int32, device=dev)
        tile_expert = torch.empty(cap // tile, dtype=torch.int32, device=dev)
        pair_slot = torch.empty(P, dtype=torch.int32, device=dev)
        ops.moe_align(experts, s.experts, tile, slots, tile_expert, pair_slot)
        act = torch.empty(cap, s.ff, device=dev, dtype=h.dtype)
        ops.expert_gemm(act, h, self.w_up, slots, tile_expert, tile, s.top, True)
        y = torch.empty(cap, self.hidden, device=dev, dtype=h.dtype)
        ops.expert_gemm(y, act, self.w_down, slots, tile_expert, tile, 0, False)
        return y, pair_slot

    def _packed_ok(self, h: torch.Tensor, P: int) -> bool:
        s = self.spec
        return (getattr(self.ops, "name", "") == "hip" and h.dtype == torch.bfloat16 and s.experts <= 128
                and self.hidden % 256 == 0 and s.ff % 256 == 0
                and P >= MOE_PACKED_MIN_PAIRS_PER_EXPERT * s.experts and not torch.cuda.is_current_stream_capturing())

    def _forward_packed(self, h: torch.Tensor, experts: torch.Tensor, P: int):
        """Large bf16 batches: the experts as two launches of the packed-layout grouped GEMM (token rows
        gathered through the slot table inside the first one, squared ReLU in its epilogue)."""
        from ..ops import gemm

        s, dev = self.spec, h.device
        op = self.ops._op  # the core kernel library
        E, H, ff = s.experts, self.hidden, s.ff
        if self.packed is None:
            pu = torch.empty(E, -(-ff // 128) * 128 * H, dtype=h.dtype, device=dev)
            pd = torch.empty(E, -(-H // 128) * 128 * ff, dtype=h.dtype, device=dev)
            op.pack_decode_weight(pu, self.w_up, False)
            op.pack_decode_weight(pd, self.w_down, False)
            self.packed = (pu, pd)
        tile = 128 * gemm.PW_WM
        cap = -(-(P + E * (tile - 1)) // tile) * tile
        slots = torch.empty(cap, dtype=torch.int32, device=dev)
        tile_expert = torch.empty(cap // tile, dtype=torch.int32, device=dev)
        ntiles = torch.empty(1, dtype=torch.int32, device=dev)
        pair_slot = torch.empty(P, dtype=torch.int32, device=dev)
        op.moe_align(experts, E, tile, slots, tile_expert, ntiles, pair_slot, None)
        pu, pd = self.packed
        act = torch.empty(cap, ff, dtype=h.dtype, device=dev)
        op.prefill_gemm_packed_grouped(act, h, pu, ff, 4, tile_expert, ntiles, gemm.PW_WM, gemm.PW_RW, slots, s.top)
        y = torch.empty(cap, H, dtype=h.dtype, device=dev)
        op.prefill_gemm_packed_grouped(y, act, pd, H, 0, tile_expert, ntiles, gemm.PW_WM, gemm.PW_RW)
        return y, pair_slot


def _linear32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x . w^T with a 32-bit result (inputs of the recurrences' decays stay 32-bit)."""
    if x.dtype == torch.float32:
        return F.linear(x, w)
    if x.is_cuda:
        return torch.mm(x, w.t(), out_dtype=torch.float32)
    return F.linear(x.float(), w.float())


def _rand(gen, *shape, std=1.0):
    return torch.randn(*shape, generator=gen) * std


class WindowAttention:
    cache_dim = property(lambda self: self.spec.cache_dim)
    state_shapes = None
    side_weight, side_rows, side_out = "w_in", 0, None

    def __init__(self, spec: WindowAttentionSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.eps, self.device, self.dtype, self.ops = spec, hidden, eps, device, dtype, ops
        self.w_in = None     # [q | k | v | gate, hidden] (q alone when the layer reads another layer's cache)
        self.b_in = None     # [same] or None
        self.q_norm = self.k_norm = None   # fp32 [heads * dim], [kv_heads * dim]; [dim] each with head_norm
        self.w_o = None      # [hidden, heads * vdim]
        self.b_o = None
        self.lam = 0.0       # differential attention: weight of the second map
        self.sink_w = None   # fp32 [heads]: learned sink logits (``sink_weights``)
        half = spec.rot_dims // 2
        i = torch.arange(half, dtype=torch.float32)
        # f_i = base^(-2i / dims), 32-bit
        self.inv_freq = torch.pow(torch.tensor(spec.rot_base, dtype=torch.float32),
                                  -2.0 * i / max(spec.rot_dims, 1)).to(device)
        self.gate_off = spec.q_size + spec.cache_dim if spec.gate else -1
        assert spec.maps in (1, 2) and not (spec.gate and spec.kv_from is not None)

    @property
    def out_size(self) -> int:
        return self.spec.heads * self.spec.vdim

    def _in_names(self):
        return ["q"] + (["k", "v"] if self.spec.kv_from is None else [])

    def load(self, get, prefix: str):
        s, dt, dev = self.spec, self.dtype, self.device
        names = self._in_names()
        self.w_in = torch.cat([get(prefix + n) for n in names + (["g"] if s.gate else [])], 0).to(dev, dt).contiguous()
        if s.bias:
            b = [get(prefix + n + ".b") for n in names] + ([torch.zeros(s.heads)] if s.gate else [])
            self.b_in = torch.cat([x.float() for x in b]).to(dev, dt).contiguous()
        if s.qk_norm or s.head_norm:
            self.q_norm = get(prefix + "q.norm").to(dev, torch.float32)
            if s.kv_from is None:
                self.k_norm = get(prefix + "k.norm").to(dev, torch.float32)
        if s.maps == 2:
            # lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number for the layer (32-bit)
            lq1, lk1, lq2, lk2 = (get(prefix + n).to(torch.float32) for n in ("lq1", "lk1", "lq2", "lk2"))
            self.lam = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + torch.tensor(s.diff))
        if s.sink_weights:
            self.sink_w = get(prefix + "sink").to(dev, torch.float32).contiguous()
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()
        if s.out_bias:
            self.b_o = get(prefix + "o.b").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden
        t = {"q": _rand(gen, s.q_size, H, std=std * 4), "o": _rand(gen, H, self.out_size, std=std)}
        if s.kv_from is None:
            t.update({"k": _rand(gen, s.k_size, H, std=std * 4), "v": _rand(gen, s.v_size, H, std=std * 4)})
        if s.gate:
            t["g"] = _rand(gen, s.heads, H, std=std * 4)
        if s.bias:
            t.update({n + ".b": _rand(gen, t[n].shape[0], std=0.3) for n in self._in_names()})
        if s.out_bias:
            t["o.b"] = _rand(gen, H, std=0.3)
        if s.qk_norm:
            t.update({"q.norm": 1.0 + 0.2 * _rand(gen, s.q_size), "k.norm": 1.0 + 0.2 * _rand(gen, s.k_size)})
        if s.head_norm:
            t.update({"q.norm": 1.0 + 0.2 * _rand(gen, s.dim), "k.norm": 1.0 + 0.2 * _rand(gen, s.dim)})
        if (s.qk_norm or s.head_norm) and s.kv_from is not None:
            del t["k.norm"]
        if s.maps == 2:
            t.update({n: _rand(gen, s.dim, std=0.2) for n in ("lq1", "lk1", "lq2", "lk2")})
        if s.sink_weights:
            t["sink"] = _rand(gen, s.heads)
        return t

    def mix(self, h, meta, cache, state, out, out_scale: float = 1.0):
        """Head outputs (before the output projection), times ``out_scale``, into ``out`` [T, heads * vdim]
        (a column slice of a wider buffer is fine)."""
        s, ops = self.spec, self.ops
        proj = F.linear(h, self.w_in, self.b_in)
        _side(self, proj)
        ops.attn_prepare(proj, cache, meta, self.inv_freq, s, self.q_norm, self.k_norm, self.eps)
        ops.window_attention(out, proj, cache, meta, s, self.gate_off, out_scale, self.lam, self.eps, self.sink_w)
        return out

    def forward(self, h, meta, cache, state):
        out = torch.empty(h.shape[0], self.out_size, device=h.device, dtype=h.dtype)
        return F.linear(self.mix(h, meta, cache, state, out), self.w_o, self.b_o)


class Wkv:
    cache_dim = 0
    input32 = True      # forward reads the 32-bit stream itself, not its rounding to the activation type
    BLENDS = ("r", "k", "v", "g", "w")
    STEP_MAX_DIM, STEP_MAX_RANK = 256, 4096   # sizes the one-row-per-sequence kernel takes

    def __init__(self, spec: WkvSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.eps, self.device, self.dtype, self.ops = spec, hidden, eps, device, dtype, ops
        self.mu = None      # fp32 [5, hidden]: blend weights of r, k, v, gate, decay
        self.w_in_t = None  # [4, hidden, heads * dim]: r, k, v, gate (transposed for the batched product)
        self.w1 = None      # [rank, hidden]
        self.w2 = None      # [heads * dim, rank]
        self.w0 = self.u = self.norm = None   # fp32 [heads * dim]
        self.w_o = None

    @property
    def out_size(self) -> int:
        return self.spec.size

    def state_shapes(self, slots: int):
        s = self.spec
        return [(slots, s.heads, s.dim, s.dim), (slots, self.hidden)]

    def load(self, get, prefix: str):
        dt, dev = self.dtype, self.device
        self.mu = torch.stack([get(prefix + "mu." + n).float() for n in self.BLENDS]).to(dev).contiguous()
        self.w_in_t = torch.stack([get(prefix + n) for n in ("r", "k", "v", "g")]).to(dev, dt).transpose(1, 2).contiguous()
        self.w1 = get(prefix + "w1").to(dev, dt).contiguous()
        self.w2 = get(prefix + "w2").to(dev, dt).contiguous()
        self.w0 = get(prefix + "w0").to(dev, torch.float32).reshape(-1).contiguous()
        self.u = get(prefix + "u").to(dev, torch.float32).reshape(-1).contiguous()
        self.norm = get(prefix + "norm").to(dev, torch.float32)
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H, N = self.spec, self.hidden, self.spec.size
        rank = s.decay_rank or max(8, N // 8)
        t = {n: _rand(gen, N, H, std=std * 4) for n in ("r", "k", "v", "g")}
        t.update({"mu." + n: torch.rand(H, generator=gen) for n in self.BLENDS})
        t.update({"w1": _rand(gen, rank, H, std=std * 4), "w2": _rand(gen, N, rank, std=0.5), "w0": _rand(gen, N) - 0.5,
                  "u": _rand(gen, s.heads, s.dim, std=0.5), "norm": 1.0 + 0.2 * _rand(gen, N), "o": _rand(gen, H, N, std=std)})
        return t

    def forward(self, x, meta, cache, state):
        """``x``: the 32-bit rows of the step."""
        s, ops = self.spec, self.ops
        T = x.shape[0]
        mixed = torch.empty(5, T, self.hidden, device=x.device, dtype=self.dtype)
        ops.token_shift(mixed, x, state[1], self.mu, meta)
        proj = torch.bmm(mixed[:4], self.w_in_t)                       # [4, T, heads * dim]: r, k, v, gate
        low = F.linear(mixed[4], self.w1)
        out = torch.empty(T, s.size, device=x.device, dtype=self.dtype)
        if meta.max_q == 1 and s.dim <= self.STEP_MAX_DIM and low.shape[1] <= self.STEP_MAX_RANK:
            # every sequence brings one row (decode steps): bottleneck, recurrence, norm and gate in one launch
            ops.wkv_step(out, state[0], proj, low, self.w2, self.w0, self.u, self.norm, s, self.eps, meta)
            return F.linear(out, self.w_o)
        ops.activation(low, low, "tanh")
        wl = _linear32(low, self.w2)
        ops.wkv(out, state[0], proj, wl, self.w0, self.u, self.norm, s, self.eps, meta)
        return F.linear(out, self.w_o)


class GatedDelta:
    cache_dim = 0

    def __init__(self, spec: GatedDeltaSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.eps, self.device, self.dtype, self.ops = spec, hidden, eps, device, dtype, ops
        self.w_in = None      # [q | k | v | beta | decay | gate, hidden]
        self.conv_w = None    # fp32 [conv channels, taps]
        self.a_log = self.dt_bias = None  # fp32 [heads]
        self.norm = None      # fp32 [vdim]
        self.w_o = None

    @property
    def out_size(self) -> int:
        return self.spec.heads * self.spec.vdim

    def state_shapes(self, slots: int):
        s = self.spec
        return [(slots, s.heads, s.dim, s.vdim), (slots, max(s.conv - 1, 1), s.conv_channels)]

    def load(self, get, prefix: str):
        dt, dev = self.dtype, self.device
        self.w_in = torch.cat([get(prefix + n) for n in ("q", "k", "v", "b", "a", "g")], 0).to(dev, dt).contiguous()
        self.conv_w = torch.cat([get(prefix + n + ".conv") for n in ("q", "k", "v")], 0).to(dev, torch.float32).contiguous()
        self.a_log = get(prefix + "A_log").to(dev, torch.float32)
        self.dt_bias = get(prefix + "dt_bias").to(dev, torch.float32)
        self.norm = get(prefix + "norm").to(dev, torch.float32)
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden
        qk = s.kv_heads * s.dim
        t = {"q": _rand(gen, qk, H, std=std * 4), "k": _rand(gen, qk, H, std=std * 4),
             "v": _rand(gen, self.out_size, H, std=std * 4), "b": _rand(gen, s.heads, H, std=std * 4),
             "a": _rand(gen, s.heads, H, std=std * 4), "g": _rand(gen, self.out_size, H, std=std * 4),
             "A_log": _rand(gen, s.heads, std=0.5) - 1.0, "dt_bias": _rand(gen, s.heads, std=0.5),
             "norm": 1.0 + 0.2 * _rand(gen, s.vdim), "o": _rand(gen, H, self.out_size, std=std)}
        for n, c in (("q", qk), ("k", qk), ("v", self.out_size)):
            t[n + ".conv"] = _rand(gen, c, s.conv, std=0.5)
        return t

    def mix(self, h, meta, cache, state, out, out_scale: float = 1.0):
        assert out_scale == 1.0
        proj = F.linear(h, self.w_in)
        self.ops.gated_delta(out, state, proj, self.conv_w, self.a_log, self.dt_bias, self.norm, self.spec, self.eps, meta)
        return out

    def forward(self, h, meta, cache, state):
        out = torch.empty(h.shape[0], self.out_size, device=h.device, dtype=h.dtype)
        return F.linear(self.mix(h, meta, cache, state, out), self.w_o)


class DeltaRule:
    cache_dim = 0

    def __init__(self, spec: DeltaRuleSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.eps, self.device, self.dtype, self.ops = spec, hidden, eps, device, dtype, ops
        self.w_in = None    # [r | k | v | a | g | decay bottleneck, hidden]
        self.w2 = None      # [heads * dim, rank]
        self.a_b = self.w0 = self.norm = None   # fp32 [heads * dim]
        self.w_o = None

    @property
    def out_size(self) -> int:
        return self.spec.size

    def state_shapes(self, slots: int):
        s = self.spec
        return [(slots, s.heads, s.dim, s.dim)]

    def load(self, get, prefix: str):
        dt, dev = self.dtype, self.device
        self.w_in = torch.cat([get(prefix + n) for n in ("r", "k", "v", "a", "g", "w1")], 0).to(dev, dt).contiguous()
        self.w2 = get(prefix + "w2").to(dev, dt).contiguous()
        self.a_b = get(prefix + "a.b").to(dev, torch.float32)
        self.w0 = get(prefix + "w0").to(dev, torch.float32)
        self.norm = get(prefix + "norm").to(dev, torch.float32)
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H, N = self.spec, self.hidden, self.spec.size
        rank = s.decay_rank or max(8, N // 8)
        t = {n: _rand(gen, N, H, std=std * 4) for n in ("r", "k", "v", "a", "g")}
        t.update({"w1": _rand(gen, rank, H, std=std * 4), "w2": _rand(gen, N, rank, std=0.5), "w0": _rand(gen, N),
                  "a.b": _rand(gen, N, std=0.5), "norm": 1.0 + 0.2 * _rand(gen, N), "o": _rand(gen, H, N, std=std)})
        return t

    def mix(self, h, meta, cache, state, out, out_scale: float = 1.0):
        N, ops = self.spec.size, self.ops
        proj = F.linear(h, self.w_in)
        low = torch.empty(h.shape[0], self.w2.shape[1], device=h.device, dtype=h.dtype)
        ops.activation(low, proj[:, 5 * N:], "tanh")
        wl = _linear32(low, self.w2)
        ops.delta_rule(out, state, proj, wl, self.a_b, self.w0, self.norm, self.spec, self.eps, meta, out_scale)
        return out

    def forward(self, h, meta, cache, state):
        out = torch.empty(h.shape[0], self.out_size, device=h.device, dtype=h.dtype)
        return F.linear(self.mix(h, meta, cache, state, out), self.w_o)


class MLstm:
    cache_dim = 0
    side_weight, side_rows, side_out = "w_in", 0, None

    def __init__(self, spec: MLstmSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.eps, self.device, self.dtype, self.ops = spec, hidden, eps, device, dtype, ops
        self.w_in = None     # [q | k | v | gate, hidden]
        self.w_if = None     # [input gate (heads) | forget gate (heads), hidden]; its product is 32-bit
        self.b_if = None     # fp32 [2 * heads]
        self.norm = None     # fp32 [heads * vdim]
        self.w_o = None

    @property
    def out_size(self) -> int:
        return self.spec.out_size

    def state_shapes(self, slots: int):
        """Matrix state, normaliser and running maximum of the log gates per sequence slot and head."""
        s = self.spec
        return [(slots, s.heads, s.dim, s.vdim), (slots, s.heads, s.dim), (slots, s.heads)]

    def load(self, get, prefix: str):
        dt, dev = self.dtype, self.device
        self.w_in = torch.cat([get(prefix + n) for n in ("q", "k", "v", "g")], 0).to(dev, dt).contiguous()
        self.w_if = torch.cat([get(prefix + "i"), get(prefix + "f")], 0).to(dev, dt).contiguous()
        self.b_if = torch.cat([get(prefix + "i.b").float(), get(prefix + "f.b").float()]).to(dev).contiguous()
        self.norm = get(prefix + "norm").to(dev, torch.float32).contiguous()
        self.w_o = get(prefix + "o").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden
        qk = s.heads * s.dim
        return {"q": _rand(gen, qk, H, std=std * 4), "k": _rand(gen, qk, H, std=std * 4),
                "v": _rand(gen, s.out_size, H, std=std * 4), "g": _rand(gen, s.out_size, H, std=std * 4),
                "i": _rand(gen, s.heads, H, std=std * 8), "f": _rand(gen, s.heads, H, std=std * 8),
                "i.b": _rand(gen, s.heads), "f.b": _rand(gen, s.heads) + 2.0,
                "norm": 1.0 + 0.2 * _rand(gen, s.out_size), "o": _rand(gen, H, s.out_size, std=std)}

    def forward(self, h, meta, cache, state):
        s = self.spec
        proj = F.linear(h, self.w_in)
        _side(self, proj)
        gates = _linear32(h, self.w_if)                                # [T, 2 * heads], 32-bit
        out = torch.empty(h.shape[0], s.out_size, device=h.device, dtype=h.dtype)
        self.ops.mlstm(out, state, proj, gates, self.b_if, self.norm, s, self.eps, meta)
        return F.linear(out, self.w_o)


class ParallelMixer:
    """left_scale * left(h) + right_scale * right(h): both halves write their scaled head outputs
    into one [T, left | right] buffer; one GEMM with the concatenated output weights sums them."""

    def __init__(self, spec: ParallelMixerSpec, hidden: int, eps: float, device, dtype, ops):
        self.spec, self.hidden, self.device, self.dtype, self.ops = spec, hidden, device, dtype, ops
        self.left = make_mixer(spec.left, hidden, eps, device, dtype, ops)
        self.right = make_mixer(spec.right, hidden, eps, device, dtype, ops)
        self.w_o = None      # [hidden, left out | right out]

    @property
    def cache_dim(self) -> int:
        assert not (self.left.cache_dim and self.right.cache_dim), "one paged cache per layer run"
        return self.left.cache_dim or self.right.cache_dim

    def state_shapes(self, slots: int):
        assert not (self.left.state_shapes and self.right.state_shapes), "one state per layer run"
        f = self.left.state_shapes or self.right.state_shapes
        return f(slots) if f else []

    def load(self, get, prefix: str):
        self.left.load(get, prefix + "left.")
        self.right.load(get, prefix + "right.")
        self.w_o = torch.cat([self.left.w_o, self.right.w_o], 1).contiguous()
        self.left.w_o = self.right.w_o = None

    def init_random(self, gen, std: float):
        t = {"left." + k: v for k, v in self.left.init_random(gen, std).items()}
        t.update({"right." + k: v for k, v in self.right.init_random(gen, std).items()})
        return t

    def forward(self, h, meta, cache, state):
        a, b = self.left.out_size, self.right.out_size
        buf = torch.empty(h.shape[0], a + b, device=h.device, dtype=h.dtype)
        self.left.mix(h, meta, cache, state, buf[:, :a], self.spec.left_scale)
        self.right.mix(h, meta, cache, state, buf[:, a:], self.spec.right_scale)
        return F.linear(buf, self.w_o)


class DenseFF:
    side_weight, side_rows, side_out = "w_up", 0, None

    def __init__(self, spec: DenseFFSpec, hidden: int, device, dtype, ops, eps: float = 0.0):
        self.spec, self.hidden, self.device, self.dtype, self.ops, self.eps = spec, hidden, device, dtype, ops, eps
        self.w_up = self.w_down = None
        self.c0 = self.c1 = 0.0     # xielu: softplus(p), 1/2 + softplus(q)
        self.coef = None            # polynorm: fp32 [4] = a, b, c, e

    def load(self, get, prefix: str):
        dt, dev = self.dtype, self.device
        self.w_up = get(prefix + "up").to(dev, dt).contiguous()
        self.w_down = get(prefix + "down").to(dev, dt).contiguous()
        if self.spec.act == "xielu":
            sp = F.softplus(get(prefix + "act").to(torch.float32))
            self.c0, self.c1 = float(sp[0]), float(torch.tensor(0.5) + sp[1])
        if self.spec.act == "polynorm":
            self.coef = get(prefix + "act").to(dev, torch.float32).contiguous()

    def init_random(self, gen, std: float):
        t = {"up": _rand(gen, self.spec.ff, self.hidden, std=std * 4), "down": _rand(gen, self.hidden, self.spec.ff, std=std)}
        if self.spec.act == "xielu":
            t["act"] = _rand(gen, 2, std=0.5)
        if self.spec.act == "polynorm":
            t["act"] = _rand(gen, 4, std=0.5)
        return t

    def forward(self, h):
        up = F.linear(h, self.w_up)
        _side(self, up)
        ff = self.spec.ff
        if self.spec.act == "polynorm":
            act = torch.empty(h.shape[0], ff, device=h.device, dtype=h.dtype)
            self.ops.polynorm(act, up[:, :ff], self.coef, self.eps)
            return F.linear(act, self.w_down)
        if self.side_rows:
            act = torch.empty(h.shape[0], ff, device=h.device, dtype=h.dtype)
            self.ops.activation(act, up[:, :ff], self.spec.act, self.c0, self.c1)
            return F.linear(act, self.w_down)
        self.ops.activation(up, up, self.spec.act, self.c0, self.c1)
        return F.linear(up, self.w_down)


class RoutedMoE:
    """``forward`` returns the parts of the mixture's output, (ye, pair_slot, ids, wts, experts, h, shared),
    which the residual update (``add_normed``) combines: row ``pair_slot[t * top + j]`` of ``ye`` is the
    output of token t's j-th choice ``ids[t, j]`` (a value >= experts is an identity expert: the token's
    own input), weighted ``wts[t, j]``; ``shared`` is the shared expert's output or None."""

    side_weight, side_rows, side_out = "ws_gu", 0, None

    def __init__(self, spec: RoutedMoESpec, hidden: int, device, dtype, ops):
        self.spec, self.hidden, self.device, self.dtype, self.ops = spec, hidden, device, dtype, ops
        self.w_router = None      # [experts + identity, hidden]
        self.correction = None    # fp32 [experts + identity]
        self.w_gu = None          # [E, 2 * ff, hidden]: gate rows, then up rows
        self.w_down = None        # [E, hidden, ff]
        self.ws_gu = self.ws_down = None   # the shared expert's [2 * shared_ff, hidden], [hidden, shared_ff]
        self.packed = None        # (gate | up, down) in the packed grouped-GEMM layout, made at the first large batch

    def load(self, get, prefix: str):
        s, dt, dev = self.spec, self.dtype, self.device
        self.w_router = get(prefix + "router").to(dev, dt).contiguous()
        self.correction = get(prefix + "correction").to(dev, torch.float32).contiguous()
        self.w_gu = torch.stack([torch.cat([get(f"{prefix}e{e}.gate"), get(f"{prefix}e{e}.up")], 0)
                                 for e in range(s.experts)]).to(dev, dt).contiguous()
        self.w_down = torch.stack([get(f"{prefix}e{e}.down") for e in range(s.experts)]).to(dev, dt).contiguous()
        if s.shared_ff:
            self.ws_gu = torch.cat([get(prefix + "shared.gate"), get(prefix + "shared.up")], 0).to(dev, dt).contiguous()
            self.ws_down = get(prefix + "shared.down").to(dev, dt).contiguous()

    def init_random(self, gen, std: float):
        s, H = self.spec, self.hidden
        n = s.experts + s.identity
        t = {"router": _rand(gen, n, H, std=std * 8), "correction": _rand(gen, n, std=0.1)}
        for e in range(s.experts):
            t.update({f"e{e}.gate": _rand(gen, s.ff, H, std=std * 4), f"e{e}.up": _rand(gen, s.ff, H, std=std * 4),
                      f"e{e}.down": _rand(gen, H, s.ff, std=std * 4)})
        if s.shared_ff:
            t.update({"shared.gate": _rand(gen, s.shared_ff, H, std=std * 4), "shared.up": _rand(gen, s.shared_ff, H, std=std * 4),
                      "shared.down": _rand(gen, H, s.shared_ff, std=std * 4)})
        return t

    def forward(self, h: torch.Tensor):
        s, ops = self.spec, self.ops
        T, dev = h.shape[0], h.device
        ids = torch.empty(T, s.top, dtype=torch.int32, device=dev)
        wts = torch.empty(T, s.top, dtype=torch.float32, device=dev)
        ops.route_topk(ids, wts, _linear32(h, self.w_router), self.correction, s.top, s.scale, s.experts,
                       s.groups, s.keep_groups, s.renorm)
        # the identity experts share one bucket (s.experts) that no GEMM tile serves
        P, nb = T * s.top, s.experts + (1 if s.identity else 0)
        if self._packed_ok(h, P, nb):
            ye, pair_slot = self._experts_packed(h, ids, P, nb)
            return ye, pair_slot, ids, wts, s.experts, h, self._shared(h)
        tile = MOE_TILE_LARGE if P >= 4 * MOE_TILE_LARGE * nb else MOE_TILE
        cap = -(-(P + nb * (tile - 1)) // tile) * tile
        slots = torch.empty(cap, dtype=torch.int32, device=dev)
        tile_expert = torch.empty(cap // tile, dtype=torch.int32, device=dev)
        pair_slot = torch.empty(P, dtype=torch.int32, device=dev)
        ops.moe_align(ids.view(-1), nb, tile, slots, tile_expert, pair_slot)
        act = torch.empty(cap, s.ff, device=dev, dtype=h.dtype)
        ops.expert_gemm(act, h, self.w_gu, slots, tile_expert, tile, s.top, 2)      # silu(gate) * up in the epilogue
        ye = torch.empty(cap, self.hidden, device=dev, dtype=h.dtype)
        ops.expert_gemm(ye, act, self.w_down, slots, tile_expert, tile, 0, 0)
        return ye, pair_slot, ids, wts, s.experts, h, self._shared(h)

    def _shared(self, h: torch.Tensor):
        """The shared expert's output (None without one); the side projection rides on its gate | up GEMM."""
        n = self.spec.shared_ff
        if not n and not self.side_rows:
            return None
        g = F.linear(h, self.ws_gu)
        _side(self, g)
        if not n:
            return None
        a = torch.empty(h.shape[0], n, device=h.device, dtype=h.dtype)
        self.ops.activation(a, g[:, :2 * n], "silu_mul")
        return F.linear(a, self.ws_down)

    def _packed_ok(self, h: torch.Tensor, P: int, nb: int) -> bool:
        from ..ops import core_built

        s = self.spec
        return (getattr(self.ops, "name", "") == "hip" and h.dtype == torch.bfloat16 and nb <= 128 and core_built()
                and self.hidden % 256 == 0 and s.ff % 256 == 0
                and P >= MOE_PACKED_MIN_PAIRS_PER_EXPERT * nb and not torch.cuda.is_current_stream_capturing())

    def _experts_packed(self, h: torch.Tensor, ids: torch.Tensor, P: int, nb: int):
        """Large bf16 batches: the experts as two launches of the packed-layout grouped GEMM of the dense
        families' MoE prefill (token rows gathered through the slot table inside the first one, the SiLU gate
        in its epilogue). The identity bucket sorts last, so the GEMMs simply stop before its tiles."""
        from ..ops import gemm

        s, dev = self.spec, h.device
        op = self.ops._op  # the core kernel library
        E, H, ff = s.experts, self.hidden, s.ff
        if self.packed is None:
            pgu = torch.empty(E, 2 * ff * H, dtype=h.dtype, device=dev)
            pd = torch.empty(E, -(-H // 128) * 128 * ff, dtype=h.dtype, device=dev)
            op.pack_decode_weight(pgu, self.w_gu, True)
            op.pack_decode_weight(pd, self.w_down, False)
            self.packed = (pgu, pd)
        tile = 128 * gemm.PW_WM
        cap = -(-(P + nb * (tile - 1)) // tile) * tile
        slots = torch.empty(cap, dtype=torch.int32, device=dev)
        tile_expert = torch.empty(cap // tile, dtype=torch.int32, device=dev)
        ntiles = torch.empty(1, dtype=torch.int32, device=dev)
        pair_slot = torch.empty(P, dtype=torch.int32, device=dev)
        op.moe_align(ids.view(-1), nb, tile, slots, tile_expert, ntiles, pair_slot, None)
        if nb > E:   # tiles of experts with weights
            ntiles = ((tile_expert >= 0) & (tile_expert < E)).sum(dtype=torch.int32).view(1)
        pgu, pd = self.packed
        act = torch.empty(cap, ff, dtype=h.dtype, device=dev)
        op.prefill_gemm_packed_grouped(act, h, pgu, 2 * ff, 2, tile_expert, ntiles, gemm.PW_WM, gemm.PW_RW, slots, s.top)
        ye = torch.empty(cap, H, dtype=h.dtype, device=dev)
        op.prefill_gemm_packed_grouped(ye, act, pd, H, 0, tile_expert, ntiles, gemm.PW_WM, gemm.PW_RW)
        return ye, pair_slot


def make_ff(spec, hidden: int, device, dtype, ops, eps: float = 0.0):
    """The weight holder of a feed-forward spec that takes no token ids."""
    if isinstance(spec, DenseFFSpec):
        return DenseFF(spec, hidden, device, dtype, ops, eps)
    if isinstance(spec, RoutedMoESpec):
        return RoutedMoE(spec, hidden, device, dtype, ops)
    raise NotImplementedError(type(spec).__name__)


def make_mixer(spec, hidden: int, eps: float, device, dtype, ops):
    """The weight holder of a mixer spec (the layer-list designs' common factory)."""
    if isinstance(spec, WindowAttentionSpec):
        return WindowAttention(spec, hidden, eps, device, dtype, ops)
    if isinstance(spec, WkvSpec):
        return Wkv(spec, hidden, eps, device, dtype, ops)
    if isinstance(spec, GatedDeltaSpec):
        return GatedDelta(spec, hidden, eps, device, dtype, ops)
    if isinstance(spec, DeltaRuleSpec):
        return DeltaRule(spec, hidden, eps, device, dtype, ops)
    if isinstance(spec, MLstmSpec):
        return MLstm(spec, hidden, eps, device, dtype, ops)
    if isinstance(spec, ParallelMixerSpec):
        return ParallelMixer(spec, hidden, eps, device, dtype, ops)
    if isinstance(spec, LatentAttentionSpec):
        return LatentAttention(spec, hidden, eps, device, dtype, ops)
    if isinstance(spec, MinGRUSpec):
        return MinGRU(spec, hidden, eps, device, dtype, ops)
    raise NotImplementedError(type(spec).__name__)
