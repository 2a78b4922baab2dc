"""hipserve op library.

``KernelOps`` calls the hand-written gfx950 kernels in ``hipserve/_C.so``
(``torch.ops.hipserve.*``) and, for the layer-list decoders, ``hipserve/_C_seq.so`` and
``hipserve/_C_delta.so`` and ``hipserve/_C_cell.so`` (``torch.ops.hipserve_seq.*``, ``torch.ops.hipserve_delta.*``, ``torch.ops.hipserve_cell.*``); each library is loaded at the first use of one of its kernels. ``ReferenceOps`` is the plain-PyTorch oracle used by
the CPU plumbing engine and by the numerics tests. The choice is made ONCE, when
an engine is built for a device — never per call. On a GPU device the native
library is mandatory: a missing/unloadable ``_C.so`` raises instead of silently
falling back to PyTorch.
"""
from __future__ import annotations

import os
import threading

import torch

from . import reference as ref

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_LIB = os.path.join(_PKG, "_C.so")
_LIB_SEQ = os.path.join(_PKG, "_C_seq.so")  # the layer-list decoders' kernels (torch.ops.hipserve_seq)
_LIB_DELTA = os.path.join(_PKG, "_C_delta.so")  # ... window attention / delta rules (torch.ops.hipserve_delta)
_LIB_CELL = os.path.join(_PKG, "_C_cell.so")  # ... gated parallel blocks, mLSTM, PolyNorm (torch.ops.hipserve_cell)
_lock = threading.Lock()
_loaded = False
_loaded_seq = False
_loaded_delta = False
_loaded_cell = False


def library_path() -> str:
    return _LIB


def load_library(build_if_missing: bool = False) -> str:
    """Load hipserve/_C.so into torch.ops (idempotent). Raises if unavailable."""
    global _loaded
    with _lock:
        if _loaded:
            return _LIB
        if not os.path.exists(_LIB) and build_if_missing:
            from .._build import build_kernels

            build_kernels()
        if not os.path.exists(_LIB):
            raise RuntimeError(
                f"hipserve native kernels not built ({_LIB} missing): run `python -m hipserve._build`")
        torch.ops.load_library(_LIB)
        _loaded = True
        return _LIB


def load_seq_library() -> str:
    """Load hipserve/_C_seq.so into torch.ops (idempotent); built first when it is missing
    (a few hipcc seconds: four kernel files)."""
    global _loaded_seq
    with _lock:
        if _loaded_seq:
            return _LIB_SEQ
        if not os.path.exists(_LIB_SEQ):
            from .._build import build_kernels

            build_kernels(lib="seq")
        torch.ops.load_library(_LIB_SEQ)
        _loaded_seq = True
        return _LIB_SEQ


def load_delta_library() -> str:
    """Load hipserve/_C_delta.so into torch.ops (idempotent); built first when it is missing."""
    global _loaded_delta
    with _lock:
        if _loaded_delta:
            return _LIB_DELTA
        if not os.path.exists(_LIB_DELTA):
            from .._build import build_kernels

            build_kernels(lib="delta")
        torch.ops.load_library(_LIB_DELTA)
        _loaded_delta = True
        return _LIB_DELTA


def load_cell_library() -> str:
    """Load hipserve/_C_cell.so into torch.ops (idempotent); built first when it is missing."""
    global _loaded_cell
    with _lock:
        if _loaded_cell:
            return _LIB_CELL
        if not os.path.exists(_LIB_CELL):
            from .._build import build_kernels

            build_kernels(lib="cell")
        torch.ops.load_library(_LIB_CELL)
        _loaded_cell = True
        return _LIB_CELL


def core_built() -> bool:
    """True when hipserve/_C.so exists (loaded or not): callers that only PREFER a core kernel ask this, so
    that a model which can do without never triggers the core library's build."""
    return _loaded or os.path.exists(_LIB)


def native_available() -> bool:
    try:
        load_library()
        return True
    except Exception:
        return False


class KernelOps:
    """gfx950 HIP kernels (all outputs written in place; graph-capturable)."""

    name = "hip"

    def __init__(self):
        self._core = None
        self._seq_ops = None
        self._delta_ops = None
        self._cell_ops = None
        # the library whose copy of the shared kernels runs ("seq" / "delta" / "cell"): a model sets it to the one
        # its mixers load anyway, so it never builds or loads another
        self.norm_library = "seq"

    @property
    def _op(self):
        """torch.ops.hipserve, loaded at the first use of a core kernel (a missing _C.so raises there)."""
        if self._core is None:
            load_library(build_if_missing=os.environ.get("HIPSERVE_BUILD_ON_DEMAND") == "1")
            self._core = torch.ops.hipserve
        return self._core

    @property
    def _seq(self):
        if self._seq_ops is None:
            load_seq_library()
            self._seq_ops = torch.ops.hipserve_seq
        return self._seq_ops

    @property
    def _delta(self):
        if self._delta_ops is None:
            load_delta_library()
            self._delta_ops = torch.ops.hipserve_delta
        return self._delta_ops

    @property
    def _cell(self):
        if self._cell_ops is None:
            load_cell_library()
            self._cell_ops = torch.ops.hipserve_cell
        return self._cell_ops

    @property
    def _latent_lib(self):
        """The library whose copy of the latent-attention kernels runs."""
        return self._cell if self.norm_library == "cell" else self._seq

    @property
    def _window_lib(self):
        """The library whose copy of the window attention, router and activation kernels runs."""
        return self._cell if self.norm_library == "cell" else self._delta

    def rmsnorm(self, out, x, w, eps, out8=None):
        """out8: (e4m3 [rows, hidden] uint8, scales fp32 [rows]) per-token FP8 copy of out."""
        self._op.rmsnorm(out, x, w, eps, *(out8 if out8 is not None else (None, None)))
        return out

    def fused_add_rmsnorm(self, out, x, residual, w, eps, out8=None):
        self._op.fused_add_rmsnorm(out, x, residual, w, eps, *(out8 if out8 is not None else (None, None)))
        return out

    def silu_and_mul(self, out, x):
        self._op.silu_and_mul(out, x)
        return out

    def gelu_and_mul(self, out, x):
        self._op.gelu_and_mul(out, x)
        return out

    def qk_rmsnorm(self, qkv, q_w, k_w, nq, nkv, D, eps):
        self._op.qk_rmsnorm(qkv, q_w, k_w, nq, nkv, D, eps)

    def fill_uniform(self, out, row0, col0, gcols, key, scale):
        self._op.fill_uniform(out, row0, col0, gcols, key, scale)
        return out

    def rope_cache(self, qkv, positions, slots, cos_sin, k_cache, v_cache, nq, nkv, D, mode):
        self._op.rope_cache(qkv, positions, slots, cos_sin, k_cache, v_cache, nq, nkv, D, mode)

    def paged_decode(self, out, q, k_cache, v_cache, block_tables, context_lens, tmp_out, tmp_ml,
                     nq, nkv, part_size, scale, window=0, out16=None):
        self._op.paged_decode(out, q, k_cache, v_cache, block_tables, context_lens, tmp_out, tmp_ml,
                              nq, nkv, part_size, scale, window, out16)
        return out

    def prefill_attention(self, out, q, k_cache, v_cache, block_tables, cu_q, ctx_lens, tiles,
                          nq, nkv, scale, window=0):
        self._op.prefill_attention(out, q, k_cache, v_cache, block_tables, cu_q, ctx_lens, tiles,
                                   nq, nkv, scale, window)
        return out

    def sample(self, out_tok, out_lp, logits, temperature, top_k, top_p, seeds, steps, two_rounds=True):
        """two_rounds=False: no row combines top-k with top-p (the multi-CU sampler's
        second fine-histogram round is then a no-op and is not launched)."""
        self._op.sample(out_tok, out_lp, logits, temperature, top_k, top_p, seeds, steps, two_rounds)

    def penalty_apply(self, logits, slot, pres, freq, rep, counts, seen):
        self._op.penalty_apply(logits, slot, pres, freq, rep, counts, seen)

    def penalty_update(self, tok, slot, counts, seen):
        self._op.penalty_update(tok, slot, counts, seen)

    def penalty_init(self, counts, seen, slots, off, n_prompt, toks):
        self._op.penalty_init(counts, seen, slots, off, n_prompt, toks)

    def top_logprobs(self, logits, nreq, out_ids, out_lp):
        self._op.top_logprobs(logits, nreq, out_ids, out_lp)

    # ---- vision tower (csrc/kernels/vision.hip)
    def layernorm(self, out, x, w, b, eps, residual=None):
        self._op.layernorm(out, x, w, b, residual, eps)
        return out

    def gelu_(self, x, tanh):
        self._op.gelu_(x, tanh)
        return x

    VISION_TILE = 128  # query rows per attention workgroup (4 waves x 32)

    def vision_meta(self, geo, nh, D):
        """(cu_seqlens, tiles) device tensors of an image batch for vision_attention."""
        import numpy as np

        cu = geo.cu_seqlens
        tiles = np.array([(s, r) for s in range(len(cu) - 1) for r in range(0, int(cu[s + 1] - cu[s]),
                                                                          self.VISION_TILE)], np.int32)
        dev = torch.device("cuda", torch.cuda.current_device())
        return (torch.from_numpy(cu.astype(np.int32)).to(dev), torch.from_numpy(tiles.reshape(-1, 2)).to(dev))

    def vision_attention(self, out, qkv, cos_sin, cu_seqlens, nh, D, scale, meta=None):
        cu, tiles = meta
        self._op.vision_attention(out, qkv, cos_sin, cu, tiles, nh, D, scale)
        return out


    # ---- layer-list decoders (csrc/kernels/seq/*.hip; bf16 or true fp32 activations)
    def scaled_add_group_rmsnorm(self, out, residual, w, groups, eps, mix=None, ls1=None, y=None, pair_slot=None,
                                 top=0, ls2=None, extra=None):
        lib = self._delta if self.norm_library == "delta" else self._seq
        lib.scaled_add_group_rmsnorm(out, residual, w, groups, eps, mix, ls1, y, pair_slot, top, ls2, extra)
        return out

    def latent_prepare(self, cq, cache, proj, positions, slots, q_norm, kv_norm, inv_freq, q_rank, kv_rank,
                       rot_dim, eps):
        self._latent_lib.latent_prepare(cq, cache, proj, positions, slots, q_norm, kv_norm, inv_freq, q_rank, kv_rank,
                                 rot_dim, eps)

    LATENT_PREFILL_TQ = 4  # tokens per workgroup of a prompt portion (x up to 4 heads = 16 waves)
    # bf16 runs the MFMA kernel (HIPSERVE_LATENT_MFMA=0: the generic kernel, as fp32 does)
    LATENT_MFMA = os.environ.get("HIPSERVE_LATENT_MFMA", "1") != "0"
    LATENT_DECODE_RUN = 128  # keys per run of a decode row (a multiple of 32; 64 measured slower)

    def latent_query_in_place(self, dtype, kv_rank, rot_dim) -> bool:
        """True when ``latent_attention`` wants the absorbed queries as bf16 rows of the cached width
        ([heads, T, kv_rank + rot_dim], the rotary part left for it to fill) instead of fp32 [heads, T, kv_rank]."""
        return dtype == torch.bfloat16 and self.LATENT_MFMA and bool(self._latent_lib.latent_attention_mfma_ok(kv_rank, rot_dim))

    def latent_attention(self, o_lat, q_abs, q, proj, cache, meta, inv_freq, heads, dim, rot_dim, kv_rank,
                         gate_off, scale, window):
        """Prompt portions (the step's first sequences) run several tokens per workgroup, decode
        rows one token per workgroup."""
        nseq = meta.seq_ctx.shape[0]
        nd = meta.num_decode
        npf, Tp = nseq - nd, meta.num_prefill_tokens
        if (q.dtype == torch.bfloat16 and self.LATENT_MFMA and self._latent_lib.latent_attention_mfma_ok(kv_rank, rot_dim)):
            # bf16: the matrix-core kernel; decode rows split their keys into runs merged by a reduce kernel
            if q_abs.dtype == torch.bfloat16:  # the absorption GEMM wrote the rows in place (latent_query_in_place)
                qc, q_abs = q_abs, None
            else:
                qc = torch.empty(heads, q.shape[0], kv_rank + rot_dim, device=q.device, dtype=q.dtype)
            fill = True
            if npf:
                self._latent_lib.latent_attention_mfma(o_lat, qc, q_abs, q, proj, meta.positions, cache, meta.seq_cu,
                                                meta.seq_ctx, meta.seq_bt, 0, npf, Tp, inv_freq, heads, dim, rot_dim,
                                                kv_rank, gate_off, scale, window, 1, 0, None, None, 0, fill)
                fill = False
            if nd:
                span = min(window, meta.max_ctx or window) if window > 0 else meta.max_ctx
                part = self.LATENT_DECODE_RUN
                while -(-span // part) > 64:
                    part *= 2
                nparts = max(1, -(-span // part))
                ws_acc = ws_ml = None
                if nparts > 1:
                    ws_acc = torch.empty(nparts, heads, nd, kv_rank, device=q.device, dtype=torch.float32)
                    ws_ml = torch.empty(nparts, heads, nd, 2, device=q.device, dtype=torch.float32)
                self._latent_lib.latent_attention_mfma(o_lat, qc, q_abs, q, proj, meta.positions, cache, meta.seq_cu,
                                                meta.seq_ctx, meta.seq_bt, npf, nseq, nd, inv_freq, heads, dim, rot_dim,
                                                kv_rank, gate_off, scale, window, nparts, part, ws_acc, ws_ml, Tp, fill)
            return
        for s0, s1, rows, tq in ((0, npf, Tp, self.LATENT_PREFILL_TQ), (npf, nseq, nd, 1)):
            if s1 > s0:
                self._latent_lib.latent_attention(o_lat, q_abs, q, proj, cache, meta.seq_cu, meta.seq_ctx, meta.seq_bt,
                                           s0, s1, rows, tq, inv_freq, heads, dim, rot_dim, kv_rank, gate_off,
                                           scale, window)

    def mingru_scan(self, y, state, proj, b_z, b_x, meta):
        self._seq.mingru_scan(y, state, proj, b_z, b_x, meta.seq_cu, meta.seq_ctx, meta.seq_state, meta.max_q)

    def attn_prepare(self, proj, cache, meta, inv_freq, sp, q_norm, k_norm, eps):
        mode = 1 if sp.qk_norm else 2 if sp.head_norm else 0
        own_kv = sp.kv_from is None   # else the layer reads another layer's cache: only q is prepared
        self._window_lib.attn_prepare(proj, cache if own_kv else None, meta.positions, meta.slot_mapping, inv_freq, sp.heads,
                                 sp.kv_heads, sp.maps, sp.dim, sp.vdim, q_norm if mode else None,
                                 k_norm if mode and own_kv else None, mode, sp.v_norm, eps)

    WINDOW_PREFILL_TQ = 4  # tokens per workgroup of a prompt portion (x the query heads of one key/value head)
    # bf16 runs the MFMA kernel (HIPSERVE_WINDOW_MFMA=0: the generic kernel, as fp32 does)
    WINDOW_MFMA = os.environ.get("HIPSERVE_WINDOW_MFMA", "1") != "0"
    WINDOW_DECODE_RUN = 128  # keys per run of a decode row (a multiple of 32)

    def window_attention(self, out, proj, cache, meta, sp, gate_off, out_scale=1.0, lam=0.0, eps=0.0, sink_w=None):
        """Prompt portions (the step's first sequences) run several tokens per workgroup, decode
        rows one token per workgroup. Two maps per head (``sp.maps`` = 2): ``lam`` weighs the second
        map, the head output is divided by its root mean square (``eps``) and scaled by 1 - ``sp.diff``.
        ``sink_w``: fp32 [heads] learned sink logits (None: 0)."""
        nseq = meta.seq_ctx.shape[0]
        nd = meta.num_decode
        npf, Tp = nseq - nd, meta.num_prefill_tokens
        diff = (sp.maps, lam, 1.0 - sp.diff, eps, sp.keep_first, sp.softcap, sink_w)
        if (proj.dtype == torch.bfloat16 and self.WINDOW_MFMA
                and self._window_lib.window_attention_mfma_ok(sp.dim, sp.vdim, out.stride(0), out.storage_offset(), sp.maps)):
            # bf16: the matrix-core kernel; decode rows split their keys into runs merged by a reduce kernel
            args = (sp.heads, sp.kv_heads, sp.dim, sp.vdim, gate_off, sp.scale, sp.window, sp.sink, out_scale)
            if npf:
                self._window_lib.window_attention_mfma(out, proj, cache, meta.seq_cu, meta.seq_ctx, meta.seq_bt, 0, npf, Tp,
                                                *args, 1, 0, None, None, 0, *diff)
            if nd:
                # keys a row can see: its window and the kept first keys behind it
                reach = sp.window + sp.keep_first
                span = min(reach, meta.max_ctx or reach) if sp.window > 0 else meta.max_ctx
                part = self.WINDOW_DECODE_RUN
                if span >= 16 * part:   # long runs of keys: fewer, longer runs per row (measured at 2k and 8k keys)
                    part *= 2
                while -(-span // part) > 64:
                    part *= 2
                nparts = max(1, -(-span // part))
                ws_acc = ws_ml = None
                if nparts > 1:
                    ws_acc = torch.empty(nparts, sp.heads * sp.maps, nd, sp.vdim, device=proj.device, dtype=torch.float32)
                    ws_ml = torch.empty(nparts, sp.heads * sp.maps, nd, 2, device=proj.device, dtype=torch.float32)
                self._window_lib.window_attention_mfma(out, proj, cache, meta.seq_cu, meta.seq_ctx, meta.seq_bt, npf, nseq, nd,
                                                *args, nparts, part, ws_acc, ws_ml, Tp, *diff)
            return
        for s0, s1, rows, tq in ((0, npf, Tp, self.WINDOW_PREFILL_TQ), (npf, nseq, nd, 1)):
            if s1 > s0:
                self._window_lib.window_attention(out, proj, cache, meta.seq_cu, meta.seq_ctx, meta.seq_bt, s0, s1, rows, tq,
                                           sp.heads, sp.kv_heads, sp.dim, sp.vdim, gate_off, sp.scale, sp.window,
                                           sp.sink, out_scale, *diff)

    def gated_delta(self, y, state, proj, conv_w, a_log, dt_bias, norm_w, sp, eps, meta):
        T = proj.shape[0]
        scratch = torch.empty(T * (2 * sp.kv_heads * sp.dim + 2 * sp.heads * sp.vdim + 2 * sp.heads),
                              device=proj.device, dtype=torch.float32)
        self._delta.gated_delta(y, state[0], state[1], proj, conv_w, a_log, dt_bias, norm_w, meta.seq_cu, meta.seq_ctx,
                              meta.seq_state, scratch, sp.heads, sp.kv_heads, sp.dim, sp.vdim, sp.conv, eps)

    def delta_rule(self, out, state, proj, wl, a_b, w0, norm_w, sp, eps, meta, out_scale=1.0):
        scratch = torch.empty(proj.shape[0] * 7 * sp.size, device=proj.device, dtype=torch.float32)
        self._delta.delta_rule(out, state[0], proj, wl, a_b, w0, norm_w, meta.seq_cu, meta.seq_ctx, meta.seq_state,
                             scratch, sp.heads, sp.dim, eps, out_scale)

    ACTIVATIONS = {"tanh": 0, "xielu": 1, "relu2": 2, "silu_mul": 3}

    def activation(self, out, x, kind, c0=0.0, c1=0.0):
        self._window_lib.activation(out, x, self.ACTIVATIONS[kind], c0, c1)
        return out

    def add_normed(self, out, residual, y, w, eps, moe=None):
        if moe is None:
            self._delta.add_normed(out, residual, w, eps, y, None, None, None, None, 0, None, None)
        else:
            ye, pair_slot, ids, wts, E, h, shared = moe
            self._delta.add_normed(out, residual, w, eps, None, ye, pair_slot, ids, wts, E, h, shared)
        return out

    def token_shift(self, out, x, state, mu, meta):
        self._delta.token_shift(out, x, state, mu, meta.seq_cu, meta.seq_ctx, meta.seq_state)

    def wkv(self, out, state, proj, wl, w0, u, norm_w, sp, eps, meta):
        scratch = torch.empty(proj.shape[1] * (5 * sp.size + sp.heads), device=proj.device, dtype=torch.float32)
        self._delta.wkv(out, state, proj, wl, w0, u, norm_w, meta.seq_cu, meta.seq_ctx, meta.seq_state, scratch,
                        sp.heads, sp.dim, eps)

    def wkv_step(self, out, state, proj, low, w2, w0, u, norm_w, sp, eps, meta):
        """``wkv`` for steps in which every sequence has one row (``meta.max_q`` == 1), the decay bottleneck's
        tanh and up-projection included (``low``: its output before the tanh): one launch."""
        self._delta.wkv_step(out, state, proj, low, w2, w0, u, norm_w, meta.seq_cu, meta.seq_ctx, meta.seq_state,
                             sp.heads, sp.dim, eps)

    ROUTER_MAX_OUTPUTS = 256

    def route_topk(self, ids, wts, logits, correction, top, scale, E, groups=1, keep_groups=1, renorm=False):
        if logits.shape[1] > self.ROUTER_MAX_OUTPUTS or groups > 64:
            # more router outputs than a wave holds: device-side torch ops
            ref.route_topk(ids, wts, logits, correction, top, scale, E, groups, keep_groups, renorm)
            return
        self._window_lib.route_topk(ids, wts, logits.contiguous(), correction, top, scale, E, groups, keep_groups, renorm)

    # ---- parallel blocks with gated sublayer results, mLSTM, PolyNorm (csrc/kernels/seq/gated_block.hip, mlstm.hip,
    # elementwise.hip)
    def gated_add_norms(self, out1, out2, residual, w1, w2, eps, first=None, second=None):
        """``first`` / ``second``: (y, g, b) of a sublayer, y its result rows or, for a mixture of experts,
        (ye, pair_slot, wts, shared)."""
        y1, g1, b1 = first if first is not None else (None, None, None)
        y2, g2, b2 = second if second is not None else (None, None, None)
        parts = (None, None, None, None)
        if isinstance(y2, tuple):
            parts, y2 = y2, None
        self._cell.gated_add_norms(out1, out2, residual, w1, w2, eps, y1, g1, b1, y2, g2, b2, *parts)

    def polynorm(self, out, x, coef, eps):
        self._cell.polynorm(out, x, coef, eps)
        return out

    def gate_mul(self, out, x, gate):
        self._cell.gate_mul(out, x, gate)
        return out

    def mlstm(self, out, state, proj, gates, b_if, norm_w, sp, eps, meta):
        scratch = torch.empty(proj.shape[0] * sp.heads * (2 * sp.dim + 2 * sp.vdim + 6), device=proj.device,
                              dtype=torch.float32)
        self._cell.mlstm(out, state[0], state[1], state[2], proj, gates, b_if, norm_w, meta.seq_cu, meta.seq_ctx,
                         meta.seq_state, scratch, sp.heads, sp.dim, sp.vdim, sp.gate_cap, eps, meta.max_q == 1)

    @property
    def _moe_lib(self):
        """The library whose copy of the expert alignment and expert GEMMs runs (the one the model loads anyway)."""
        if self.norm_library == "cell":
            return self._cell
        return self._delta if self.norm_library == "delta" else self._seq

    def moe_align(self, experts, E, tile, slots, tile_expert, pair_slot):
        if E <= 128:
            self._moe_lib.moe_align(experts, E, tile, slots, tile_expert, pair_slot)
            return
        # more experts than the alignment kernel's LDS tables hold: the same layout from device-side
        # sort / scan ops (no host round trip)
        ex = experts.long()
        P = ex.numel()
        order = torch.argsort(ex, stable=True)
        counts = torch.bincount(ex, minlength=E)
        padded = (counts + tile - 1) // tile * tile
        ends = torch.cumsum(padded, 0)
        first = torch.cumsum(counts, 0) - counts           # rank of each expert's first pair in `order`
        e_sorted = ex[order]
        pos = (ends - padded)[e_sorted] + torch.arange(P, device=ex.device) - first[e_sorted]
        slots.fill_(-1)
        slots[pos] = order.to(torch.int32)
        pair_slot[order] = pos.to(torch.int32)
        t = torch.arange(tile_expert.numel(), device=ex.device) * tile
        te = torch.searchsorted(ends, t, right=True)
        tile_expert.copy_(torch.where(te < E, te, torch.full_like(te, -1)).to(torch.int32))

    def expert_gemm(self, out, x, w, slots, tile_expert, tile, gather_k, act):
        """act: False / 0 none, True / 1 squared ReLU, 2: w = [gate rows; up rows], out = silu(gate) * up."""
        self._moe_lib.expert_gemm(out, x, w, slots, tile_expert, tile, gather_k, int(act))


class ReferenceOps:
    """PyTorch reference path (CPU plumbing engine / numerics oracle)."""

    name = "reference"

    def fill_uniform(self, out, row0, col0, gcols, key, scale):
        return ref.fill_uniform(out, row0, col0, gcols, key, scale)

    def rmsnorm(self, out, x, w, eps, out8=None):
        assert out8 is None, "the FP8 copy is a HIP-kernel output"
        out.copy_(ref.rmsnorm(x, w, eps))
        return out

    def fused_add_rmsnorm(self, out, x, residual, w, eps, out8=None):
        assert out8 is None, "the FP8 copy is a HIP-kernel output"
        y, r = ref.fused_add_rmsnorm(x, residual, w, eps)
        residual.copy_(r)
        out.copy_(y)
        return out

    def silu_and_mul(self, out, x):
        out.copy_(ref.silu_and_mul(x))
        return out

    def gelu_and_mul(self, out, x):
        out.copy_(ref.gelu_and_mul(x))
        return out

    def qk_rmsnorm(self, qkv, q_w, k_w, nq, nkv, D, eps):
        ref.qk_rmsnorm(qkv, q_w, k_w, nq, nkv, D, eps)

    def rope_cache(self, qkv, positions, slots, cos_sin, k_cache, v_cache, nq, nkv, D, mode):
        ref.rope_cache(qkv, positions, slots, cos_sin, k_cache, v_cache, nq, nkv, D, mode)

    def paged_decode(self, out, q, k_cache, v_cache, block_tables, context_lens, tmp_out, tmp_ml,
                     nq, nkv, part_size, scale, window=0, out16=None):
        B = context_lens.shape[0]
        D = k_cache.shape[3]
        out[:B, : nq * D].copy_(ref.paged_decode(q, k_cache, v_cache, block_tables, context_lens,
                                                 nq, nkv, scale, window).view(B, nq * D))
        return out

    def prefill_attention(self, out, q, k_cache, v_cache, block_tables, cu_q, ctx_lens, tiles,
                          nq, nkv, scale, window=0):
        D = k_cache.shape[3]
        T = int(cu_q[-1])
        out[:T, : nq * D].copy_(ref.prefill_attention(q, k_cache, v_cache, block_tables, cu_q,
                                                      ctx_lens, nq, nkv, scale, window).view(T, nq * D))
        return out

    def penalty_apply(self, logits, slot, pres, freq, rep, counts, seen):
        ref.penalty_apply(logits, slot, pres, freq, rep, counts, seen)

    def penalty_update(self, tok, slot, counts, seen):
        ref.penalty_update(tok, slot, counts, seen)

    def penalty_init(self, counts, seen, slots, off, n_prompt, toks):
        ref.penalty_init(counts, seen, slots, off, n_prompt, toks)

    def top_logprobs(self, logits, nreq, out_ids, out_lp):
        ref.top_logprobs(logits, nreq, out_ids, out_lp)

    # ---- vision tower (Qwen3-VL ViT)
    def layernorm(self, out, x, w, b, eps, residual=None):
        if residual is None:
            out.copy_(ref.layernorm(x, w, b, eps))
        else:
            y, r = ref.add_layernorm(x, residual, w, b, eps)
            residual.copy_(r)
            out.copy_(y)
        return out

    def gelu_(self, x, tanh):
        x.copy_(ref.gelu(x, tanh))
        return x

    def vision_attention(self, out, qkv, cos_sin, cu_seqlens, nh, D, scale, meta=None):
        ref.vision_rope(qkv, cos_sin, nh, D)
        out.copy_(ref.vision_attention(qkv, cu_seqlens, nh, D, scale))
        return out

    # ---- layer-list decoders (models/mixers.py)
    def scaled_add_group_rmsnorm(self, out, residual, w, groups, eps, mix=None, ls1=None, y=None, pair_slot=None,
                                 top=0, ls2=None, extra=None):
        ref.scaled_add_group_rmsnorm(out, residual, w, groups, eps, mix, ls1, y, pair_slot, top, ls2, extra)
        return out

    def latent_prepare(self, cq, cache, proj, positions, slots, q_norm, kv_norm, inv_freq, q_rank, kv_rank,
                       rot_dim, eps):
        ref.latent_prepare(cq, cache, proj, positions, slots, q_norm, kv_norm, inv_freq, q_rank, kv_rank, rot_dim, eps)

    def latent_attention(self, o_lat, q_abs, q, proj, cache, meta, inv_freq, heads, dim, rot_dim, kv_rank,
                         gate_off, scale, window):
        ref.latent_attention(o_lat, q_abs, q, proj, cache, meta.seq_cu, meta.seq_ctx, meta.seq_bt, inv_freq,
                             heads, dim, rot_dim, kv_rank, gate_off, scale, window)

    def latent_query_in_place(self, dtype, kv_rank, rot_dim) -> bool:
        return False

    def mingru_scan(self, y, state, proj, b_z, b_x, meta):
        ref.mingru_scan(y, state, proj, b_z, b_x, meta.seq_cu, meta.seq_ctx, meta.seq_state)

    def moe_align(self, experts, E, tile, slots, tile_expert, pair_slot):
        ref.moe_align(experts, E, tile, slots, tile_expert, pair_slot)

    def expert_gemm(self, out, x, w, slots, tile_expert, tile, gather_k, act):
        ref.expert_gemm(out, x, w, slots, tile_expert, tile, gather_k, int(act))

    def attn_prepare(self, proj, cache, meta, inv_freq, sp, q_norm, k_norm, eps):
        ref.attn_prepare(proj, cache, meta.positions, meta.slot_mapping, inv_freq, sp, q_norm, k_norm, eps)

    def window_attention(self, out, proj, cache, meta, sp, gate_off, out_scale=1.0, lam=0.0, eps=0.0, sink_w=None):
        ref.window_attention(out, proj, cache, meta.seq_cu, meta.seq_ctx, meta.seq_bt, sp, gate_off, out_scale, lam, eps,
                             sink_w)

    def gated_add_norms(self, out1, out2, residual, w1, w2, eps, first=None, second=None):
        ref.gated_add_norms(out1, out2, residual, w1, w2, eps, first, second)

    def polynorm(self, out, x, coef, eps):
        ref.polynorm(out, x, coef, eps)
        return out

    def gate_mul(self, out, x, gate):
        ref.gate_mul(out, x, gate)
        return out

    def mlstm(self, out, state, proj, gates, b_if, norm_w, sp, eps, meta):
        ref.mlstm(out, state[0], state[1], state[2], proj, gates, b_if, norm_w, sp, eps, meta.seq_cu, meta.seq_ctx,
                  meta.seq_state)

    def add_normed(self, out, residual, y, w, eps, moe=None):
        ref.add_normed(out, residual, y, w, eps, moe)
        return out

    def token_shift(self, out, x, state, mu, meta):
        ref.token_shift(out, x, state, mu, meta.seq_cu, meta.seq_ctx, meta.seq_state)

    def wkv(self, out, state, proj, wl, w0, u, norm_w, sp, eps, meta):
        ref.wkv(out, state, proj, wl, w0, u, norm_w, sp, eps, meta.seq_cu, meta.seq_ctx, meta.seq_state)

    def wkv_step(self, out, state, proj, low, w2, w0, u, norm_w, sp, eps, meta):
        t = torch.tanh(low.float()).to(low.dtype)
        wl = torch.nn.functional.linear(t.float(), w2.float())
        ref.wkv(out, state, proj, wl, w0, u, norm_w, sp, eps, meta.seq_cu, meta.seq_ctx, meta.seq_state)

    def route_topk(self, ids, wts, logits, correction, top, scale, E, groups=1, keep_groups=1, renorm=False):
        ref.route_topk(ids, wts, logits, correction, top, scale, E, groups, keep_groups, renorm)

    def gated_delta(self, y, state, proj, conv_w, a_log, dt_bias, norm_w, sp, eps, meta):
        ref.gated_delta(y, state[0], state[1], proj, conv_w, a_log, dt_bias, norm_w, sp, eps, meta.seq_cu,
                        meta.seq_ctx, meta.seq_state)

    def delta_rule(self, out, state, proj, wl, a_b, w0, norm_w, sp, eps, meta, out_scale=1.0):
        ref.delta_rule(out, state[0], proj, wl, a_b, w0, norm_w, sp, eps, meta.seq_cu, meta.seq_ctx,
                       meta.seq_state, out_scale)

    def activation(self, out, x, kind, c0=0.0, c1=0.0):
        ref.activation(out, x, kind, c0, c1)
        return out

    def sample(self, out_tok, out_lp, logits, temperature, top_k, top_p, seeds, steps, two_rounds=True):
        t, lp = ref.sample(logits, temperature, top_k, top_p, seeds, steps, bf16_row=False)
        n = t.shape[0]
        out_tok[:n].copy_(t)
        if out_lp.numel():
            out_lp[:n].copy_(lp)


def get_ops(device: torch.device | str):
    device = torch.device(device)
    if device.type == "cuda":
        return KernelOps()
    return ReferenceOps()
