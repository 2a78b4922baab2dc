"""Plain-PyTorch fp32 reference implementations of every hipserve kernel.

These are the numerics oracles for the gfx950 kernels (tests compare the HIP op
against these) and the compute path of the CPU plumbing engine (tests/CI without
a GPU). They use exactly the same tensor layouts as the kernels:

* ``k_cache [num_blocks, nkv, block_size, D]``
* ``v_cache [num_blocks, nkv, D, block_size]`` (transposed per block)
* ``cos_sin [max_pos, D]`` = ``[cos(D/2) | sin(D/2)]`` fp32
"""
from __future__ import annotations

import math

import numpy as np
import torch


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    inv = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (xf * inv * w.float()).to(x.dtype)


def fused_add_rmsnorm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, eps: float):
    """Returns (normed, new_residual); residual is rounded to x.dtype first."""
    r = (x.float() + residual.float()).to(x.dtype)
    return rmsnorm(r, w, eps), r


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    inter = x.shape[-1] // 2
    g, u = x[..., :inter].float(), x[..., inter:].float()
    return (torch.nn.functional.silu(g) * u).to(x.dtype)


def gelu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """tanh-GELU(gate) * up (Gemma GeGLU, HF gelu_pytorch_tanh)."""
    inter = x.shape[-1] // 2
    g, u = x[..., :inter].float(), x[..., inter:].float()
    return (torch.nn.functional.gelu(g, approximate="tanh") * u).to(x.dtype)


def layernorm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """LayerNorm over the last dim (fp32 statistics, x.dtype out)."""
    return torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(), eps).to(x.dtype)


def add_layernorm(x: torch.Tensor, residual: torch.Tensor, w, b, eps: float):
    """(LayerNorm(r), r) with r = residual + x rounded to x.dtype first."""
    r = (x.float() + residual.float()).to(x.dtype)
    return layernorm(r, w, b, eps), r


def gelu(x: torch.Tensor, tanh: bool) -> torch.Tensor:
    return torch.nn.functional.gelu(x.float(), approximate="tanh" if tanh else "none").to(x.dtype)


def vision_rope(qkv: torch.Tensor, cos_sin: torch.Tensor, nh: int, D: int):
    """In place: rotate-half RoPE of the q and k heads of a ViT qkv [T, 3*nh*D] with one
    fp32 table row per token ([cos(D/2) | sin(D/2)], the 2D row/column angles)."""
    T = qkv.shape[0]
    half = D // 2
    c, s = cos_sin[:T, None, :half].float(), cos_sin[:T, None, half:].float()
    for j in range(2):
        x = qkv[:, j * nh * D:(j + 1) * nh * D].view(T, nh, D)
        a, b = x[..., :half].float(), x[..., half:].float()
        x.copy_(torch.cat([a * c - b * s, b * c + a * s], -1).to(x.dtype))


def vision_attention(qkv: torch.Tensor, cu_seqlens, nh: int, D: int, scale: float) -> torch.Tensor:
    """Bidirectional attention within each segment [cu[i], cu[i+1]) of a ViT qkv
    [T, 3*nh*D] (fp32 math) -> [T, nh*D]."""
    T = qkv.shape[0]
    q = qkv[:, : nh * D].view(T, nh, D).float()
    k = qkv[:, nh * D:2 * nh * D].view(T, nh, D).float()
    v = qkv[:, 2 * nh * D:].view(T, nh, D).float()
    out = torch.empty(T, nh, D, dtype=torch.float32, device=qkv.device)
    cu = [int(x) for x in cu_seqlens]
    for a, b in zip(cu[:-1], cu[1:]):
        s = torch.einsum("qhd,khd->hqk", q[a:b], k[a:b]) * scale
        out[a:b] = torch.einsum("hqk,khd->qhd", torch.softmax(s, -1), v[a:b])
    return out.view(T, nh * D).to(qkv.dtype)


def qk_rmsnorm(qkv: torch.Tensor, q_w: torch.Tensor, k_w: torch.Tensor, nq: int, nkv: int, D: int, eps: float):
    """In place: RMSNorm over head_dim of every q head (weight q_w) and k head (k_w)."""
    T = qkv.shape[0]
    if T == 0:
        return
    q = qkv[:, : nq * D].view(T, nq, D)
    k = qkv[:, nq * D:(nq + nkv) * D].view(T, nkv, D)
    q.copy_(rmsnorm(q, q_w, eps))
    k.copy_(rmsnorm(k, k_w, eps))


def rope_cos_sin(head_dim: int, max_pos: int, theta: float, scaling: dict | None = None,
                 rotary_dim: int | None = None) -> torch.Tensor:
    """fp32 [max_pos, D] table = [cos | sin] with optional Llama-3 frequency scaling."""
    rd = rotary_dim or head_dim
    inv_freq = 1.0 / (theta ** (torch.arange(0, rd, 2, dtype=torch.float64) / rd))
    if scaling and scaling.get("rope_type", scaling.get("type")) == "llama3":
        factor = scaling["factor"]
        lo, hi = scaling.get("low_freq_factor", 1.0), scaling.get("high_freq_factor", 4.0)
        old = scaling.get("original_max_position_embeddings", 8192)
        lo_wl, hi_wl = old / lo, old / hi
        wl = 2 * math.pi / inv_freq
        smooth = (old / wl - lo) / (hi - lo)
        scaled = torch.where(wl > lo_wl, inv_freq / factor, inv_freq)
        mid = (wl <= lo_wl) & (wl >= hi_wl)
        scaled = torch.where(mid, (1 - smooth) * inv_freq / factor + smooth * inv_freq, scaled)
        inv_freq = scaled
    elif scaling and scaling.get("rope_type", scaling.get("type")) == "linear":
        inv_freq = inv_freq / scaling["factor"]
    t = torch.arange(max_pos, dtype=torch.float64)
    f = torch.outer(t, inv_freq)
    return torch.cat([f.cos(), f.sin()], dim=-1).float().contiguous()


def apply_rope(x: torch.Tensor, pos: torch.Tensor, cos_sin: torch.Tensor, mode: int) -> torch.Tensor:
    """x [T, H, D] -> rotated (fp32 math, x.dtype out)."""
    D = x.shape[-1]
    half = D // 2
    cs = cos_sin[pos.long()]  # [T, D]
    c, s = cs[:, None, :half], cs[:, None, half:]
    xf = x.float()
    if mode == 0:
        a, b = xf[..., :half], xf[..., half:]
        out = torch.cat([a * c - b * s, b * c + a * s], dim=-1)
    else:
        a, b = xf[..., 0::2], xf[..., 1::2]
        out = torch.stack([a * c - b * s, b * c + a * s], dim=-1).flatten(-2)
    return out.to(x.dtype)


def to_cache(x: torch.Tensor, dtype) -> torch.Tensor:
    """K / V rows in the cache's element type: e4m3 caches saturate to +-448 first (the
    kernels' rounding, common.h kv_store*); torch's own cast turns overflow into NaN."""
    if dtype == torch.float8_e4m3fn:
        return x.float().clamp(-448.0, 448.0).to(dtype)
    return x.to(dtype)


def rope_cache(qkv, positions, slots, cos_sin, k_cache, v_cache, nq, nkv, D, mode):
    """In-place: rotates q inside qkv, writes rotated k and raw v into the caches."""
    T = qkv.shape[0]
    if T == 0:
        return
    q = qkv[:, : nq * D].view(T, nq, D)
    k = qkv[:, nq * D:(nq + nkv) * D].view(T, nkv, D)
    v = qkv[:, (nq + nkv) * D:(nq + 2 * nkv) * D].view(T, nkv, D)
    q.copy_(apply_rope(q, positions[:T], cos_sin, mode))
    kr = apply_rope(k, positions[:T], cos_sin, mode)
    bs = k_cache.shape[2]
    sl = slots[:T].long()
    valid = sl >= 0
    if valid.any():
        sv = sl[valid]
        blk, off = sv // bs, sv % bs
        k_cache[blk, :, off, :] = to_cache(kr[valid], k_cache.dtype)
        v_cache[blk, :, :, off] = to_cache(v[valid], v_cache.dtype)


def _gather_kv(k_cache, v_cache, block_table, n):
    bs = k_cache.shape[2]
    idx = torch.arange(n, device=k_cache.device)
    blk = block_table[(idx // bs)].long()
    off = idx % bs
    k = k_cache[blk, :, off, :]          # [n, nkv, D]
    v = v_cache[blk, :, :, off]          # [n, nkv, D]
    return k, v


def paged_decode(q, k_cache, v_cache, block_tables, context_lens, nq, nkv, scale, window=0):
    """q [B, nq*D (+extra)] -> out [B, nq, D] (fp32 math). window > 0: only the
    last ``window`` keys (sliding-window layers)."""
    D = k_cache.shape[3]
    B = context_lens.shape[0]
    G = nq // nkv
    out = torch.empty(B, nq, D, dtype=q.dtype, device=q.device)
    for b in range(B):
        n = int(context_lens[b])
        k, v = _gather_kv(k_cache, v_cache, block_tables[b], n)
        if window > 0 and n > window:
            k, v = k[n - window:], v[n - window:]
        qb = q[b, : nq * D].view(nq, D).float()
        kf = k.float().repeat_interleave(G, dim=1)  # [n, nq, D]
        vf = v.float().repeat_interleave(G, dim=1)
        s = torch.einsum("hd,nhd->hn", qb, kf) * scale
        p = torch.softmax(s, dim=-1)
        out[b] = torch.einsum("hn,nhd->hd", p, vf).to(q.dtype)
    return out


def prefill_attention(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, nq, nkv, scale, window=0):
    """q [T, nq*D (+extra)] -> out [T, nq, D]; causal over absolute positions;
    window > 0: keys within ``window - 1`` positions before the query."""
    D = k_cache.shape[3]
    G = nq // nkv
    T = int(cu_q[-1])
    out = torch.empty(T, nq, D, dtype=q.dtype, device=q.device)
    for s_ in range(len(ctx_lens)):
        q0, q1 = int(cu_q[s_]), int(cu_q[s_ + 1])
        ql, ctx = q1 - q0, int(ctx_lens[s_])
        if ql == 0:
            continue
        k, v = _gather_kv(k_cache, v_cache, block_tables[s_], ctx)
        qs = q[q0:q1, : nq * D].view(ql, nq, D).float()
        kf = k.float().repeat_interleave(G, dim=1)
        vf = v.float().repeat_interleave(G, dim=1)
        s = torch.einsum("qhd,nhd->hqn", qs, kf) * scale
        qpos = torch.arange(ctx - ql, ctx, device=q.device)[:, None]
        kpos = torch.arange(ctx, device=q.device)[None, :]
        mask = kpos > qpos
        if window > 0:
            mask = mask | (kpos <= qpos - window)
        s = s.masked_fill(mask[None], float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[q0:q1] = torch.einsum("hqn,nhd->qhd", p, vf).to(q.dtype)
    return out


# ---- sampling: the same counter-based RNG as csrc/kernels/sampling.hip ----


def row_key(seed: int, step: int) -> int:
    M = (1 << 64) - 1
    x = ((seed & M) * 0x9E3779B97F4A7C15 & M) ^ (((step & M) + 0xD1B54A32D192ED03) & M) * 0xBF58476D1CE4E5B9 & M
    x ^= x >> 31
    x = x * 0x7FB5D329728EA185 & M
    x ^= x >> 27
    x = x * 0x81DADEF4BC2DD44D & M
    x ^= x >> 33
    return (x ^ (x >> 32)) & 0xFFFFFFFF


def uniform01(seed: int, step: int, n: int) -> np.ndarray:
    key = np.uint32(row_key(seed, step))
    with np.errstate(over="ignore"):
        i = np.arange(n, dtype=np.uint32)
        h = key ^ (i * np.uint32(0x9E3779B9) + np.uint32(0x7F4A7C15))
        h ^= h >> np.uint32(16)
        h *= np.uint32(0x85EBCA6B)
        h ^= h >> np.uint32(13)
        h *= np.uint32(0xC2B2AE35)
        h ^= h >> np.uint32(16)
    return (((h >> np.uint32(8)).astype(np.float64) + 0.5) / 16777216.0).astype(np.float32)


def sample(logits: torch.Tensor, temperature, top_k, top_p, seeds, steps, bf16_row: bool = True):
    """Returns (tokens int64 [B], logprobs f32 [B]) with the kernel's semantics:
    greedy if T<=1e-5; else top-k then top-p (on the top-k-renormalised mass) then
    a Gumbel-max draw with u = hash(seed, step, index). ``bf16_row`` mirrors the
    kernel, which holds an fp32 row as bf16; the CPU engine samples full fp32."""
    B, V = logits.shape
    toks = torch.empty(B, dtype=torch.long)
    lps = torch.empty(B, dtype=torch.float32)
    # the kernel holds the row as bf16 in registers: sample on bf16-rounded logits
    lf = logits.float().cpu()
    if bf16_row:
        lf = lf.to(torch.bfloat16).float()
    for r in range(B):
        x = lf[r]
        lse = torch.logsumexp(x, 0)
        t = float(temperature[r])
        if not t > 1e-5:
            i = int(torch.argmax(x))
            toks[r], lps[r] = i, float(x[i] - lse)
            continue
        keep = torch.ones(V, dtype=torch.bool)
        k = int(top_k[r])
        if 0 < k < V:
            kth = torch.topk(x, k).values[-1]
            keep &= x >= kth
        p = float(top_p[r])
        if p < 1.0:
            w = torch.exp((x - x.max()) / t) * keep
            order = torch.argsort(x, descending=True)
            cum = torch.cumsum(w[order].double(), 0)
            target = p * float(cum[-1])
            n = int(torch.searchsorted(cum, torch.tensor([target], dtype=torch.float64))[0])
            thr = x[order[min(n, V - 1)]]
            keep &= x >= thr
        u = torch.from_numpy(uniform01(int(seeds[r]), int(steps[r]), V))
        g = (x - x.max()) / t - torch.log(-torch.log(u))
        g = torch.where(keep, g, torch.full_like(g, float("-inf")))
        i = int(torch.argmax(g))
        toks[r], lps[r] = i, float(x[i] - lse)
    return toks, lps


# ----------------------------------------------------------------------------- K16
def _mix32(x: torch.Tensor) -> torch.Tensor:
    """lowbias32 on int64 tensors holding uint32 values (products wrap mod 2^64,
    the low 32 bits are exact)."""
    M = 0xFFFFFFFF
    x = x ^ (x >> 16)
    x = (x * 0x7FEB352D) & M
    x = x ^ (x >> 15)
    x = (x * 0x846CA68B) & M
    return x ^ (x >> 16)


def fill_uniform(out: torch.Tensor, row0: int, col0: int, gcols: int, key: int, scale: float):
    """Torch twin of csrc/kernels/init.hip (bit-identical): uniform(-scale, scale)
    keyed by global element coordinates, written into the 2-D view ``out``."""
    rows, cols = out.shape
    r = torch.arange(rows, dtype=torch.int64).unsqueeze(1) + row0
    c = torch.arange(cols, dtype=torch.int64).unsqueeze(0) + col0
    idx = (r * gcols + c) & 0xFFFFFFFF
    h = _mix32(_mix32(idx) ^ (key & 0xFFFFFFFF))
    u = (h >> 8).to(torch.float32) * 5.9604644775390625e-08
    v = (u - 0.5) * torch.tensor(2.0 * scale, dtype=torch.float32)
    out.copy_(v.to(torch.bfloat16).to(out.dtype))
    return out


# ---------------------------------------------------------------- penalties / logprobs
# Oracle of csrc/kernels/penalties.hip. State per slot: counts int32 [slots, V]
# (generated-token occurrences), seen int32 [slots, ceil(V/32)] bitmask (prompt or
# generated). vLLM / OpenAI order: repetition first, then frequency + presence.
def _seen_mask(seen: torch.Tensor, V: int) -> torch.Tensor:
    v = torch.arange(V, device=seen.device)
    return ((seen[:, v // 32] >> (v % 32)) & 1).bool()


def penalty_apply(logits, slot, pres, freq, rep, counts, seen):
    rows, V = logits.shape
    for r in range(rows):
        s = int(slot[r])
        p, f, q = float(pres[r]), float(freq[r]), float(rep[r])
        if s < 0 or (p == 0.0 and f == 0.0 and q == 1.0):
            continue
        l = logits[r].float()
        m = _seen_mask(seen[s:s + 1], V)[0]
        l = torch.where(m, torch.where(l > 0, l / q, l * q), l)
        c = counts[s].float()
        l = l - f * c - p * (c > 0).float()
        logits[r].copy_(l.to(logits.dtype))
    return logits


def penalty_update(tok, slot, counts, seen):
    V = counts.shape[1]
    for r in range(tok.shape[0]):
        s, t = int(slot[r]), int(tok[r])
        if s < 0 or not 0 <= t < V:
            continue
        counts[s, t] += 1
        seen[s, t // 32] |= _bit(t)


def _bit(t: int) -> int:
    b = 1 << (t % 32)
    return b - (1 << 32) if b >= (1 << 31) else b  # int32 two's complement


def penalty_init(counts, seen, slots, off, n_prompt, toks):
    V = counts.shape[1]
    for j in range(slots.shape[0]):
        s = int(slots[j])
        counts[s].zero_()
        seen[s].zero_()
        a, b, npr = int(off[j]), int(off[j + 1]), int(n_prompt[j])
        for i in range(a, b):
            t = int(toks[i])
            if not 0 <= t < V:
                continue
            seen[s, t // 32] |= _bit(t)
            if i - a >= npr:
                counts[s, t] += 1


def top_logprobs(logits, nreq, out_ids, out_lp):
    """n largest log-softmax entries per row (ties -> lowest id), K = out width.

    Exact over the whole row. The device kernel (csrc/kernels/penalties.hip
    top_logprobs) is exact too unless more than 64 keys share the bf16 bin of the n-th
    largest value: it then keeps the lowest-index 64 of them, so in a row
    with > 64 logits within one bf16 ulp of the n-th largest the two may name different
    (equally probable to bf16 precision) entries."""
    K = out_ids.shape[1]
    out_ids.fill_(-1)
    out_lp.fill_(float("-inf"))
    for r in range(logits.shape[0]):
        n = min(int(nreq[r]), K)
        if n <= 0:
            continue
        l = logits[r].float()
        ls = l - torch.logsumexp(l, 0)
        # order by (exact value desc, id asc): stable sort keeps equal values in id order
        order = torch.argsort(-l, stable=True)[:n].tolist()
        for i, v in enumerate(order):
            out_ids[r, i] = v
            out_lp[r, i] = ls[v]


# ---------------------------------------------------------------------------------
# layer-list decoders (models/mixers.py): grouped norm + residual update, latent
# attention on a paged latent cache, minGRU scan over state slots, table-routed experts

def scaled_add_group_rmsnorm(out, residual, w, groups, eps, mix=None, ls1=None, y=None, pair_slot=None, top=0,
                             ls2=None, extra=None):
    """residual (fp32, in place) += ls1 * mix + ls2 * mean_j y[pair_slot[t * top + j]] + extra;
    out = residual normalised in ``groups`` equal consecutive parts, times w."""
    T, H = residual.shape
    if mix is not None:
        residual += mix.float() * ls1.float() if ls1 is not None else mix.float()
    if y is not None:
        rows = y.float().index_select(0, pair_slot.long()).view(T, top, H)
        residual += rows.sum(1) * (1.0 / top) * ls2.float()
    if extra is not None:
        residual += extra.float()
    g = residual.view(T, groups, H // groups)
    g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((g.reshape(T, H) * w.float()).to(out.dtype))


def partial_rope(x: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """Rotate-half RoPE of the first 2 * len(inv_freq) elements of the last dim (fp32);
    pair (i, i + n): (u cos a - v sin a, v cos a + u sin a), a = pos * inv_freq[i]."""
    n = inv_freq.shape[0]
    a = pos.float().unsqueeze(-1) * inv_freq.float()
    while a.dim() < x.dim():
        a = a.unsqueeze(-2)
    c, s = a.cos(), a.sin()
    u, v = x[..., :n].float(), x[..., n:2 * n].float()
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:].float()], -1)


def latent_prepare(cq, cache, proj, positions, slots, q_norm, kv_norm, inv_freq, q_rank, kv_rank, rot_dim, eps):
    """proj rows = [q latent | kv latent | rotary key | ...]: cq = RMSNorm(q latent) * q_norm;
    cache[slot] = [RMSNorm(kv latent) * kv_norm | RoPE(rotary key)] for slots >= 0."""
    p = proj.float()
    a = p[:, :q_rank]
    cq.copy_((a * torch.rsqrt(a.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()).to(cq.dtype))
    c = p[:, q_rank:q_rank + kv_rank]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * kv_norm.float()
    kr = partial_rope(p[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim], positions, inv_freq)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok]] = row[ok]


def latent_attention(o_lat, q_abs, q, proj, cache, seq_cu, seq_ctx, seq_bt, inv_freq, heads, dim, rot_dim,
                     kv_rank, gate_off, scale, window):
    """Per sequence s with rows cu[s]..cu[s+1]-1 at positions ctx[s] - n .. ctx[s] - 1: scores of
    head h = (q_abs[h, t] . latent + RoPE(q[t, h, dim:]) . rotary key) * scale over the keys
    0 <= pos - j < window (window 0: all j <= pos), softmax, latent-space output times
    sigmoid(proj[t, gate_off + h]) (gate_off >= 0)."""
    bs = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1])
    cu = [int(v) for v in seq_cu]
    T = q.shape[0]
    qh = q.view(T, heads, dim + rot_dim)
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if a == b:
            continue
        ctx = int(seq_ctx[s])
        pos = torch.arange(ctx - (b - a), ctx, device=q.device)
        lo = 0 if window <= 0 else max(0, int(pos[0]) - window + 1)
        j = torch.arange(lo, ctx, device=q.device)
        rows = seq_bt[s].long()[j // bs] * bs + j % bs
        kv = flat[rows].float()                                  # [n_keys, kv_rank + rot_dim]
        qr = partial_rope(qh[a:b, :, dim:], pos, inv_freq)       # [n, heads, rot_dim]
        sc = torch.einsum("hnk,jk->hnj", q_abs[:, a:b].float(), kv[:, :kv_rank])
        sc = (sc + torch.einsum("nhr,jr->hnj", qr, kv[:, kv_rank:])) * scale
        d = pos[:, None] - j[None]
        ok = (d >= 0) & ((d < window) if window > 0 else (d >= 0))
        sc = sc.masked_fill(~ok, float("-inf"))
        o = torch.einsum("hnj,jk->hnk", torch.softmax(sc, -1), kv[:, :kv_rank])
        if gate_off >= 0:
            o = o * torch.sigmoid(proj[a:b, gate_off:gate_off + heads].float()).t().unsqueeze(-1)   # [heads, n, 1]
        o_lat[:, a:b] = o.to(o_lat.dtype)


def mingru_scan(y, state, proj, b_z, b_x, seq_cu, seq_ctx, seq_state):
    """proj rows = [z | x | g] pre-activations. Per sequence, from its state slot (zero when
    the step starts at position 0): S = (1 - z) S + z c, z = sigmoid(. + b_z), u = . + b_x,
    c = u + 0.5 (u >= 0) or sigmoid(u); y = S * silu(g). The slot gets the last S."""
    n = state.shape[1]
    cu = [int(v) for v in seq_cu]
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if a == b:
            continue
        slot = int(seq_state[s])
        S = state[slot].clone() if int(seq_ctx[s]) - (b - a) > 0 else torch.zeros_like(state[slot])
        p = proj[a:b].float()
        z = torch.sigmoid(p[:, :n] + b_z)
        u = p[:, n:2 * n] + b_x
        c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        g = p[:, 2 * n:]
        g = g * torch.sigmoid(g)
        for t in range(b - a):
            S = (1 - z[t]) * S + z[t] * c[t]
            y[a + t] = (S * g[t]).to(y.dtype)
        state[slot] = S


def moe_align(experts, E, tile, slots, tile_expert, pair_slot):
    """Pairs sorted by expert into tiles of ``tile`` slots: slots[pos] = pair index or -1
    (padding), tile_expert[t] = the tile's expert or -1, pair_slot[p] = the pair's slot."""
    slots.fill_(-1)
    tile_expert.fill_(-1)
    pos = 0
    ex = experts.tolist()
    for e in range(E):
        ps = [p for p, v in enumerate(ex) if v == e]
        for k, p in enumerate(ps):
            slots[pos + k] = p
            pair_slot[p] = pos + k
        nt = -(-len(ps) // tile)
        tile_expert[pos // tile:pos // tile + nt] = e
        pos += nt * tile


def expert_gemm(out, x, w, slots, tile_expert, tile, gather_k, act):
    """out[slot] = act(W[e(slot)] . x[row(slot)]); row = slots[slot] // gather_k (gather_k > 0)
    or the slot itself; act 0: none, 1: squared ReLU, 2: W = [gate rows; up rows] and
    out = silu(gate) * up (half as wide). Padding slots are left untouched."""
    sl = slots.tolist()
    te = tile_expert.tolist()
    for s, p in enumerate(sl):
        if p < 0:
            continue
        e = te[s // tile]
        if e < 0 or e >= w.shape[0]:   # a tile of the bucket that has no weights (identity experts)
            continue
        row = p // gather_k if gather_k > 0 else s
        v = w[e].float() @ x[row].float()
        if act == 1:
            v = torch.relu(v) ** 2
        elif act == 2:
            n = v.shape[0] // 2
            v = v[:n] * torch.sigmoid(v[:n]) * v[n:]
        out[s] = v.to(out.dtype)


# ---------------------------------------------------------------------------------
# windowed sink attention on a paged [keys | values] cache, the two delta-rule
# recurrences over state slots, per-head output norm + gate, elementwise activations

def _rows_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def attn_prepare(proj, cache, positions, slots, inv_freq, sp, q_norm, k_norm, eps):
    """proj rows = [q | k | v | ...] (after biases), or [q | ...] alone when the layer reads another
    layer's cache (``sp.kv_from``). In place on the q columns: the optional RMS norm (``sp.qk_norm``:
    over the whole projection, a weight per element; ``sp.head_norm``: over every head - and map -
    of ``dim`` elements, one weight of ``dim`` elements for all) and the rotation; the cache row of
    slots >= 0 gets [keys | values], keys normed and rotated alike, values divided by their per-head
    root mean square when ``sp.v_norm``."""
    T = proj.shape[0]
    nq, nk, nv = sp.q_size, sp.k_size, sp.v_size
    own_kv = sp.kv_from is None
    p = proj.float()
    q = p[:, :nq]
    k, v = (p[:, nq:nq + nk], p[:, nq + nk:nq + nk + nv]) if own_kv else (None, None)
    if sp.qk_norm:
        q = _rows_rms(q, eps) * q_norm.float()
        if own_kv:
            k = _rows_rms(k, eps) * k_norm.float()
    q = q.reshape(T, sp.heads * sp.maps, sp.dim)
    if sp.head_norm:
        q = _rows_rms(q, eps) * q_norm.float()
    proj[:, :nq] = partial_rope(q, positions, inv_freq).reshape(T, nq).to(proj.dtype)
    if not own_kv:
        return
    k = k.reshape(T, sp.kv_heads * sp.maps, sp.dim)
    if sp.head_norm:
        k = _rows_rms(k, eps) * k_norm.float()
    k = partial_rope(k, positions, inv_freq).reshape(T, nk)
    if sp.v_norm:
        v = _rows_rms(v.reshape(T, sp.kv_heads, sp.vdim), eps).reshape(T, nv)
    ok = slots >= 0
    cache.view(-1, cache.shape[-1])[slots[ok]] = torch.cat([k, v], -1).to(cache.dtype)[ok]


def window_attention(out, proj, cache, seq_cu, seq_ctx, seq_bt, sp, gate_off, out_scale, lam=0.0, eps=0.0, sink_w=None):
    """Per sequence s (rows cu[s]..cu[s+1]-1 at positions ctx[s]-n .. ctx[s]-1): head h scores
    its prepared query against the cached keys of head h // (heads / kv_heads) with
    0 <= pos - j < window or j < sp.keep_first; scores s_j = q . k * scale, then
    softcap * tanh(s_j / softcap) (softcap > 0); weights exp(s_j) / (sink + sum exp(s_j)) with
    sink = exp(sink_w[h]) (1 without weights); out[t, h * vdim ..] =
    weighted values * sigmoid(proj[t, gate_off + h]) (gate_off >= 0) * out_scale.
    ``sp.maps`` = 2: query and key heads hold [map 1 | map 2]; the head output is
    o = a1 - lam * a2 of the two maps' weighted values, o / sqrt(mean(o^2) + eps) * (1 - sp.diff)."""
    bs = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1])
    cu = [int(x) for x in seq_cu]
    H, G, M, d, dv, W = sp.heads, sp.kv_heads, sp.maps, sp.dim, sp.vdim, sp.window
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if a == b:
            continue
        ctx = int(seq_ctx[s])
        pos = torch.arange(ctx - (b - a), ctx, device=proj.device)
        lo = 0 if (W <= 0 or sp.keep_first > 0) else max(0, int(pos[0]) - W + 1)
        j = torch.arange(lo, ctx, device=proj.device)
        kv = flat[seq_bt[s].long()[j // bs] * bs + j % bs].float()
        k = kv[:, :G * M * d].view(-1, G, M * d).repeat_interleave(H // G, 1).reshape(-1, H * M, d)
        v = kv[:, G * M * d:G * M * d + G * dv].view(-1, G, dv).repeat_interleave(H // G, 1)
        v = v.repeat_interleave(M, 1)
        q = proj[a:b, :H * M * d].float().view(b - a, H * M, d)
        sc = torch.einsum("nhd,jhd->hnj", q, k) * sp.scale
        if sp.softcap > 0:
            sc = torch.tanh(sc / sp.softcap) * sp.softcap
        dd = pos[:, None] - j[None]
        ok = (dd >= 0) & (((dd < W) | (j[None] < sp.keep_first)) if W > 0 else (dd >= 0))
        sc = sc.masked_fill(~ok, float("-inf"))
        m = sc.max(-1, keepdim=True).values
        sk = 0.0   # the sink's logit: a key without a value
        if sp.sink and sink_w is not None:
            sk = sink_w.float().repeat_interleave(M).view(H * M, 1, 1)
        if sp.sink:
            m = torch.maximum(m, torch.as_tensor(sk, dtype=m.dtype, device=m.device))
        e = torch.exp(sc - m)
        den = e.sum(-1, keepdim=True) + (torch.exp(sk - m) if sp.sink else 0.0)
        o = torch.einsum("hnj,jhv->nhv", e / den, v)
        if M == 2:
            o = o.view(b - a, H, 2, dv)
            o = o[:, :, 0] - lam * o[:, :, 1]
            o = _rows_rms(o, eps) * (1.0 - sp.diff)
        if gate_off >= 0:
            o = o * torch.sigmoid(proj[a:b, gate_off:gate_off + H].float()).unsqueeze(-1)
        out[a:b] = (o * out_scale).reshape(b - a, H * dv).to(out.dtype)


def _conv_inputs(proj, conv_state, a, b, start, slot, C, taps):
    """The step's conv inputs of one sequence with the taps - 1 inputs before them in front."""
    x = proj[a:b, :C].float()
    prev = conv_state[slot][:taps - 1]
    return torch.cat([prev if start > 0 else torch.zeros_like(prev), x], 0)


def gated_delta(y, S, conv_state, proj, conv_w, a_log, dt_bias, norm_w, sp, eps, seq_cu, seq_ctx, seq_state):
    """proj rows = [q | k | v | beta | decay | gate] pre-activations. Per sequence, from its slot
    (zero when the step starts at position 0): causal conv + SiLU on q, k, v; unit q (times
    dim^-1/2) and k; S = g S; u = beta (v - S^T k); S += k u^T; o = S^T q; y = o / rms(o) *
    norm_w * silu(gate). S [slots, heads, dim, vdim], conv_state [slots, taps - 1, channels]."""
    H, G, d, dv, taps = sp.heads, sp.kv_heads, sp.dim, sp.vdim, sp.conv
    C = sp.conv_channels
    cu = [int(x) for x in seq_cu]
    w = conv_w.float()
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        n = b - a
        if n == 0:
            continue
        slot, start = int(seq_state[s]), int(seq_ctx[s]) - n
        xin = _conv_inputs(proj, conv_state, a, b, start, slot, C, taps)
        xc = sum(xin[j:j + n] * w[:, j] for j in range(taps))
        xc = xc * torch.sigmoid(xc)
        if taps > 1:
            conv_state[slot] = xin[n:]
        q = xc[:, :G * d].view(n, G, d)
        k = xc[:, G * d:2 * G * d].view(n, G, d)
        v = xc[:, 2 * G * d:].view(n, H, dv)
        q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        q, k = q.repeat_interleave(H // G, 1), k.repeat_interleave(H // G, 1)
        p = proj[a:b, C:].float()
        beta = torch.sigmoid(p[:, :H])
        g = torch.exp(-torch.exp(a_log.float()) * torch.nn.functional.softplus(p[:, H:2 * H] + dt_bias.float()))
        gate = p[:, 2 * H:].view(n, H, dv)
        st = S[slot].clone() if start > 0 else torch.zeros_like(S[slot])
        o = torch.empty(n, H, dv)
        for t in range(n):
            st = st * g[t, :, None, None]
            u = beta[t, :, None] * (v[t] - torch.einsum("hkv,hk->hv", st, k[t]))
            st = st + k[t, :, :, None] * u[:, None, :]
            o[t] = torch.einsum("hkv,hk->hv", st, q[t])
        S[slot] = st
        o = _rows_rms(o, eps) * norm_w.float() * (gate * torch.sigmoid(gate))
        y[a:b] = o.reshape(n, H * dv).to(y.dtype)


def delta_rule(out, S, proj, wl, a_b, w0, norm_w, sp, eps, seq_cu, seq_ctx, seq_state, out_scale):
    """proj rows = [r | k | v | a | g | ...] pre-activations, wl the decay bottleneck's output
    (fp32). Per head with u = unit(k): w = exp(-e^-1/2 sigmoid(wl + w0)), a = sigmoid(a + a_b),
    S = diag(w) S - (a u)(u^T S) + k v^T (both terms on the old S), o = S^T r;
    out = o / rms(o) * norm_w * sigmoid(g) * out_scale. S [slots, heads, dim(key), dim(value)]."""
    H, d = sp.heads, sp.dim
    N = H * d
    cu = [int(x) for x in seq_cu]
    for s in range(len(cu) - 1):
        a0, b0 = cu[s], cu[s + 1]
        n = b0 - a0
        if n == 0:
            continue
        slot, start = int(seq_state[s]), int(seq_ctx[s]) - n
        p = proj[a0:b0].float()
        r, k, v = (p[:, i * N:(i + 1) * N].view(n, H, d) for i in range(3))
        rem = torch.sigmoid(p[:, 3 * N:4 * N] + a_b.float()).view(n, H, d)
        gate = torch.sigmoid(p[:, 4 * N:5 * N])
        w = torch.exp(-0.6065306597126334 * torch.sigmoid(wl[a0:b0].float() + w0.float())).view(n, H, d)
        u = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
        st = S[slot].clone() if start > 0 else torch.zeros_like(S[slot])
        o = torch.empty(n, H, d)
        for t in range(n):
            uS = torch.einsum("hkv,hk->hv", st, u[t])
            st = w[t, :, :, None] * st - (rem[t] * u[t])[:, :, None] * uS[:, None, :] + k[t, :, :, None] * v[t, :, None, :]
            o[t] = torch.einsum("hkv,hk->hv", st, r[t])
        S[slot] = st
        o = _rows_rms(o, eps).reshape(n, N) * norm_w.float() * gate * out_scale
        out[a0:b0] = o.to(out.dtype)


def activation(out, x, kind, c0=0.0, c1=0.0):
    """Elementwise: ``tanh``; ``relu2`` = max(z, 0)^2; ``xielu`` with c0 = softplus(p),
    c1 = 1/2 + softplus(q): c0 z^2 + z/2 for z > 0, c1 (exp(z) - 1 - z) + z/2 otherwise;
    ``silu_mul``: x rows = [gate | up], out = silu(gate) * up (half as wide)."""
    z = x.float()
    if kind == "tanh":
        r = torch.tanh(z)
    elif kind == "relu2":
        r = torch.relu(z) ** 2
    elif kind == "silu_mul":
        n = z.shape[-1] // 2
        r = z[..., :n] * torch.sigmoid(z[..., :n]) * z[..., n:]
    elif kind == "xielu":
        zn = z.clamp(max=0.0)
        r = torch.where(z > 0, c0 * z * z + 0.5 * z, c1 * (torch.expm1(zn) - zn) + 0.5 * z)
    else:
        raise ValueError(kind)
    out.copy_(r.to(out.dtype))


# ---------------------------------------------------------------------------------
# residual update with the norm on the sublayer's output, token shift, linear attention
# with per-channel decays over state slots, softmax router with a selection correction

def add_normed(out, residual, y, w, eps, moe=None):
    """residual (fp32, in place) += y / sqrt(mean(y^2) + eps) * w; out = residual in out's dtype.
    With ``moe`` = (ye, pair_slot, ids, wts, E, h, shared) the addend is the mixture's output:
    y[t] = shared[t] + sum_j wts[t, j] * (ye[pair_slot[t * top + j]] if ids[t, j] < E else h[t])."""
    if moe is not None:
        ye, pair_slot, ids, wts, E, h, shared = moe
        T, top = ids.shape
        rows = ye.float().index_select(0, pair_slot.long().clamp(min=0)).view(T, top, -1)
        rows = torch.where((ids < E).unsqueeze(-1), rows, h.float().unsqueeze(1).expand_as(rows))
        y = (rows * wts.float().unsqueeze(-1)).sum(1)
        if shared is not None:
            y = y + shared.float()
    residual += _rows_rms(y.float(), eps) * w.float()
    out.copy_(residual.to(out.dtype))


def token_shift(out, x, state, mu, seq_cu, seq_ctx, seq_state):
    """out[s, t] = x[t] + (x[t - 1] - x[t]) * mu[s] for every blend s; the row before a step's first
    row comes from the sequence's slot (zeros at position 0); the slot gets the step's last row."""
    cu = [int(v) for v in seq_cu]
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        if a == b:
            continue
        slot = int(seq_state[s])
        first = state[slot].clone() if int(seq_ctx[s]) - (b - a) > 0 else torch.zeros_like(state[slot])
        xs = x[a:b].float()
        prev = torch.cat([first[None], xs[:-1]], 0)
        out[:, a:b] = (xs[None] + (prev - xs)[None] * mu.float()[:, None, :]).to(out.dtype)
        state[slot] = xs[-1]


def wkv(out, S, proj, wl, w0, u, norm_w, sp, eps, seq_cu, seq_ctx, seq_state):
    """proj [4, T, N] = r, k, v and the gate's pre-activation (N = heads * dim), wl the decay
    bottleneck's output (fp32 [T, N]). Per head: w = exp(-exp(wl + w0)); o = (S + diag(u) k v^T)^T r;
    S = diag(w) S + k v^T; out = o / rms(o) * norm_w * silu(gate). S [slots, heads, dim(key), dim(value)]."""
    H, d = sp.heads, sp.dim
    N = H * d
    cu = [int(x) for x in seq_cu]
    for s in range(len(cu) - 1):
        a0, b0 = cu[s], cu[s + 1]
        n = b0 - a0
        if n == 0:
            continue
        slot, start = int(seq_state[s]), int(seq_ctx[s]) - n
        r, k, v = (proj[i, a0:b0].float().view(n, H, d) for i in range(3))
        g = proj[3, a0:b0].float()
        w = torch.exp(-torch.exp(wl[a0:b0].float() + w0.float())).view(n, H, d)
        uu = u.float().view(H, d)
        st = S[slot].clone() if start > 0 else torch.zeros_like(S[slot])
        o = torch.empty(n, H, d)
        for t in range(n):
            kv = k[t, :, :, None] * v[t, :, None, :]
            o[t] = torch.einsum("hkv,hk->hv", st + uu[:, :, None] * kv, r[t])
            st = w[t, :, :, None] * st + kv
        S[slot] = st
        out[a0:b0] = (_rows_rms(o, eps).reshape(n, N) * norm_w.float() * (g * torch.sigmoid(g))).to(out.dtype)


def route_topk(ids, wts, logits, correction, top, scale, E, groups=1, keep_groups=1, renorm=False):
    """s = softmax(logits) (fp32, over all router outputs); the ``top`` outputs with the largest
    s + correction are chosen (ties: the lower index); wts = s * scale of the chosen, ids = their
    index, outputs >= E (experts without weights) all written as E. ``groups`` > 1: the outputs
    form equal groups of neighbours, a group scores its largest s + correction, and outputs
    outside the ``keep_groups`` best groups cannot be chosen. ``renorm``: the chosen s are divided
    by their sum (+ 1e-20) before the scaling."""
    s = torch.softmax(logits.float(), -1)
    c = s + correction.float()
    if groups > 1:
        T, n = c.shape
        best = c.view(T, groups, n // groups).max(-1).values
        kept = torch.argsort(-best, dim=-1, stable=True)[:, :keep_groups]
        allow = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        c = c.masked_fill(~allow.repeat_interleave(n // groups, 1), float("-inf"))
    order = torch.argsort(-c, dim=-1, stable=True)[:, :top]
    w = s.gather(1, order)
    if renorm:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    wts.copy_(w * scale)
    ids.copy_(order.clamp(max=E).to(ids.dtype))


# ---------------------------------------------------------------------------------
# parallel blocks with gated sublayer results and two single-weight norms, PolyNorm, the
# per-channel output gate of heads stored head-major, the mLSTM matrix memory over state slots

def gated_add_norms(out1, out2, residual, w1, w2, eps, first=None, second=None):
    """residual (fp32, in place) += sum over the given sublayers of sigmoid(g + b) * y, each
    ``(y, g, b)`` with y [T, H] the sublayer's result (or the parts of a mixture's output,
    ``(ye, pair_slot, wts, shared)``: y[t] = shared[t] + sum_j wts[t, j] * ye[pair_slot[t * top + j]]),
    g [T, H] its gate's pre-activation (any row stride) and b [H] the gate's bias. Then
    out1 = residual / rms * w1 and out2 = residual / rms * w2 (w: one number or H; out2 / w2 may be None)."""
    for sub in (first, second):
        if sub is None:
            continue
        y, g, b = sub
        if isinstance(y, tuple):
            ye, pair_slot, wts, shared = y
            T, top = wts.shape
            rows = ye.float().index_select(0, pair_slot.long().clamp(min=0)).view(T, top, -1)
            y = (rows * wts.float().unsqueeze(-1)).sum(1)
            if shared is not None:
                y = y + shared.float()
        residual += torch.sigmoid(g.float() + b.float()) * y.float()
    n = _rows_rms(residual, eps)
    out1.copy_((n * w1.float()).to(out1.dtype))
    if out2 is not None:
        out2.copy_((n * w2.float()).to(out2.dtype))


def polynorm(out, x, coef, eps):
    """out = a N(z) + b N(z^2) + c N(z^3) + e over every row z of x, N(u) = u / sqrt(mean(u^2) + eps),
    coef = [a, b, c, e] (fp32)."""
    z = x.float()
    a, b, c, e = (coef[i].float() for i in range(4))
    out.copy_((a * _rows_rms(z, eps) + b * _rows_rms(z * z, eps) + c * _rows_rms(z * z * z, eps) + e).to(out.dtype))


def gate_mul(out, x, gate):
    """out[t, h * d + j] = x[h, t, j] * sigmoid(gate[t, h * d + j]) for x [heads, T, d] (head-major)."""
    Hh, T, d = x.shape
    out.copy_((x.float().transpose(0, 1).reshape(T, Hh * d) * torch.sigmoid(gate.float())).to(out.dtype))


def mlstm(out, S, N, M, proj, gates, b_if, norm_w, sp, eps, seq_cu, seq_ctx, seq_state):
    """proj rows = [q | k | v | gate | ...], gates (fp32) rows = [input gate | forget gate] pre-activations per head.
    Per head, from the sequence's slot (zeros when the step starts at position 0), with
    i = cap tanh((. + b) / cap), f = logsigmoid(cap tanh((. + b) / cap)), q scaled by dim^-1/2:
      m' = max(f + m, i);  S = e^(f + m - m') S + e^(i - m') k v^T;  n likewise with k;  m = m'
      o = S^T q / (max(|n . q|, e^-m) + 1e-6)
    out = o / rms(o) per head * norm_w * sigmoid(gate). S [slots, heads, dim, vdim], N [slots, heads, dim], M [slots, heads]."""
    H, d, dv, cap = sp.heads, sp.dim, sp.vdim, sp.gate_cap
    cu = [int(x) for x in seq_cu]
    for s in range(len(cu) - 1):
        a0, b0 = cu[s], cu[s + 1]
        n = b0 - a0
        if n == 0:
            continue
        slot, start = int(seq_state[s]), int(seq_ctx[s]) - n
        p = proj[a0:b0].float()
        q = p[:, :H * d].view(n, H, d) * d ** -0.5
        k = p[:, H * d:2 * H * d].view(n, H, d)
        v = p[:, 2 * H * d:2 * H * d + H * dv].view(n, H, dv)
        gate = p[:, 2 * H * d + H * dv:2 * H * d + 2 * H * dv]
        pre = gates[a0:b0].float() + b_if.float()
        ig = cap * torch.tanh(pre[:, :H] / cap)
        fg = torch.nn.functional.logsigmoid(cap * torch.tanh(pre[:, H:] / cap))
        if start > 0:
            st, nn, mm = S[slot].clone(), N[slot].clone(), M[slot].clone()
        else:
            st, nn, mm = torch.zeros_like(S[slot]), torch.zeros_like(N[slot]), torch.zeros_like(M[slot])
        o = torch.empty(n, H, dv, device=proj.device)
        for t in range(n):
            m_new = torch.maximum(fg[t] + mm, ig[t])
            fa, fb = torch.exp(fg[t] + mm - m_new), torch.exp(ig[t] - m_new)
            st = fa[:, None, None] * st + fb[:, None, None] * k[t, :, :, None] * v[t, :, None, :]
            nn = fa[:, None] * nn + fb[:, None] * k[t]
            mm = m_new
            den = torch.maximum((nn * q[t]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
            o[t] = torch.einsum("hkv,hk->hv", st, q[t]) / den[:, None]
        S[slot], N[slot], M[slot] = st, nn, mm
        out[a0:b0] = (_rows_rms(o, eps).reshape(n, H * dv) * norm_w.float() * torch.sigmoid(gate)).to(out.dtype)
