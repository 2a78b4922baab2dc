"""Plain, slow float64 implementation of the Topezen decoder, one function per mechanism,
written from the design's equations. It reads a config DICT (the layout of a model folder's
config.json) and a dict of named tensors, and shares no code with hipserve: the tests
compare the engine against it.

Notation: x [n, width] is one sequence's residual stream, positions count from 0.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def lin(w, x):
    """Weights are stored [out, in]; rows of x are tokens."""
    return x @ w.T


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def rotate_pairs(x, pos, base, dims):
    """x [n, heads, d]: coordinates (2i, 2i+1), i < dims/2, turn by the angle pos * base^(-2i/dims)."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=F64)
    ang = pos.to(F64)[:, None] * base ** (-2.0 * i / dims)          # [n, dims/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ---------------------------------------------------------------- mixers
def latent_attention(h, w, m, eps):
    """w: the mixer's tensors by short name (dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o)."""
    n = h.shape[0]
    H, d, r, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n)
    cq = rms_unit(lin(w["dq"], h), eps) * w["dq.norm"]
    q = lin(w["uq"], cq).view(n, H, d + r)
    q_nope, q_rot = q[..., :d], q[..., d:]
    dkv = lin(w["dkv"], h)
    c = rms_unit(dkv[:, :kr], eps) * w["dkv.norm"]
    k_rot = dkv[:, kr:].view(n, 1, r)
    rot = m["rot"]
    q_rot = rotate_pairs(q_rot, pos, rot["base"], rot["dims"])
    k_rot = rotate_pairs(k_rot, pos, rot["base"], rot["dims"])
    k_nope = lin(w["uk"], c).view(n, H, d)
    v = lin(w["uv"], c).view(n, H, dv)
    sc = (torch.einsum("ihd,jhd->hij", q_nope, k_nope) + torch.einsum("ihr,jr->hij", q_rot, k_rot[:, 0])) * m["scale"]
    causal = pos[None, :] <= pos[:, None]
    sc = sc.masked_fill(~causal, -math.inf)
    o = torch.einsum("hij,jhv->ihv", torch.softmax(sc, -1), v).reshape(n, H * dv)
    o = o * sigmoid(lin(w["g"], h))
    return lin(w["o"], o)


def mlstm(h, w, m, eps, state=None):
    """Matrix memory with a running maximum; ``state`` = (S [H, d, dv], n [H, d], m [H]) carries on."""
    n = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = lin(w["q"], h).view(n, H, d) * d ** -0.5
    k = lin(w["k"], h).view(n, H, d)
    v = lin(w["v"], h).view(n, H, dv)
    ig = cap * torch.tanh((lin(w["i"], h) + w["i.b"]) / cap)                       # [n, H] log input gate
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((lin(w["f"], h) + w["f.b"]) / cap))
    if state is None:
        S, nn, mm = torch.zeros(H, d, dv, dtype=F64), torch.zeros(H, d, dtype=F64), torch.zeros(H, dtype=F64)
    else:
        S, nn, mm = (t.clone() for t in state)
    out = torch.empty(n, H, dv, dtype=F64)
    for t in range(n):
        m_new = torch.maximum(fg[t] + mm, ig[t])
        a = torch.exp(fg[t] + mm - m_new)
        b = torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        nn = a[:, None] * nn + b[:, None] * k[t]
        mm = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((nn * q[t]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
        out[t] = num / den[:, None]
    o = rms_unit(out, eps).reshape(n, H * dv) * w["norm"] * sigmoid(lin(w["g"], h))
    return lin(w["o"], o), (S, nn, mm)


def sink_attention(h, w, m, eps):
    """Grouped-query attention without positions: capped scores, a window that keeps the first
    tokens, a learned sink in the softmax denominator."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_unit(lin(w["q"], h).view(n, H, d), eps) * w["q.norm"]
    k = rms_unit(lin(w["k"], h).view(n, G, d), eps) * w["k.norm"]
    v = lin(w["v"], h).view(n, G, dv)
    k = k.repeat_interleave(H // G, 1)
    v = v.repeat_interleave(H // G, 1)
    sc = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    cap = m["softcap"]
    sc = cap * torch.tanh(sc / cap)
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    size, keep = m["mask"]["size"], m["mask"]["keep_first"]
    seen = (j <= i) & ((i - j < size) | (j < keep))
    sc = sc.masked_fill(~seen, -math.inf)
    e = torch.exp(sc)                                                    # plain exponentials: float64 holds them
    den = e.sum(-1, keepdim=True) + torch.exp(w["sink"])[:, None, None]
    o = torch.einsum("hij,jhv->ihv", e / den, v).reshape(n, H * dv)
    return lin(w["o"], o)


# ---------------------------------------------------------------- feed-forwards
def polynorm_ff(h, w, eps):
    z = lin(w["up"], h)
    a, b, c, e = w["act"]
    act = a * rms_unit(z, eps) + b * rms_unit(z ** 2, eps) + c * rms_unit(z ** 3, eps) + e
    return lin(w["down"], act)


def gated_expert(h, gate, up, down):
    z = lin(gate, h)
    return lin(down, z * sigmoid(z) * lin(up, h))


def route(h, w, r):
    """Chosen experts [n, top] and their weights [n, top]."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(lin(w["router"], h), -1)
    choice = s + w["correction"]
    g = r.get("groups")
    if g:
        per = E // g["count"]
        best = choice.view(-1, g["count"], per).max(-1).values           # [n, groups]
        kept = torch.topk(best, g["keep"], dim=-1).indices
        allow = torch.zeros_like(best, dtype=torch.bool).scatter_(1, kept, True)
        choice = choice.masked_fill(~allow.repeat_interleave(per, 1), -math.inf)
    ids = torch.topk(choice, top, dim=-1).indices
    ws = s.gather(1, ids)
    return ids, ws / (ws.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, w, f):
    ids, ws = route(h, w, f["router"])
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t].tolist(), ws[t]):
            out[t] += wt * gated_expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if f.get("shared"):
        out = out + gated_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


# ---------------------------------------------------------------- the model
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg: dict, tensors: dict, tokens, states=None, return_layers: bool = False):
    """Logits [n, vocab] of one sequence from position 0 (or, with ``states``, the recurrent layers go on
    from them; attention layers always see only ``tokens``, so use it for models without attention)."""
    W = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens)] * cfg["embedding"]["scale"]
    after, new_states = [], []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h1 = rms_unit(x, eps) * W[p + "norm1"]
        wm = sub(W, p + "mix.")
        if L["type"] == "latent_attention":
            y = latent_attention(h1, wm, L["mixer"], eps)
        elif L["type"] == "mlstm":
            y, st = mlstm(h1, wm, L["mixer"], eps, states[len(new_states)] if states else None)
            new_states.append(st)
        elif L["type"] == "attention":
            y = sink_attention(h1, wm, L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        upd = y * sigmoid(lin(W[p + "rg1"], h1) + W[p + "rg1.b"])
        f = L.get("mlp")
        if f is not None:
            h2 = rms_unit(x, eps) * W[p + "norm2"]
            wf = sub(W, p + "mlp.")
            z = polynorm_ff(h2, wf, eps) if f["kind"] == "dense" else moe_ff(h2, wf, f)
            upd = upd + z * sigmoid(lin(W[p + "rg2"], h2) + W[p + "rg2.b"])
        x = x + upd
        after.append(x.clone())
    logits = lin(W["head"], rms_unit(x, eps) * W["final.norm"])
    if return_layers:
        return logits, torch.stack(after), new_states
    return logits
