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


# ------------------------------------------------------------------ small configs and random weights
def latent_layer(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=10, kv_rank=12, scale=None, base=10000.0, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale or (dim + rot_dim) ** -0.5, "rot": {"base": base, "dims": rot_dim}}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def mlstm_layer(heads=2, dim=8, vdim=12, gate_cap=10.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": gate_cap}, "mlp": mlp}


def attn_layer(heads=4, kv_heads=2, dim=8, vdim=12, scale=None, softcap=15.0, size=11, keep_first=3, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5,
         "softcap": softcap, "mask": {"size": size, "keep_first": keep_first}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=12, count=3, keep=2, shared=20):
    f = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def make_config(layers, width=32, vocab=96, eps=1e-5, scale=3.0):
    return {"architecture": "Topezen", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps},
            "vocab": vocab, "width": width}


def make_weights(cfg, seed=0, gain=1.0):
    """Random checkpoint tensors (values representable in bf16) under the design's names."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def lin(o, i):
        return rnd(o, i, std=gain / math.sqrt(i))

    W = {"embed": rnd(V, Wd, std=1.0 / cfg["embedding"]["scale"]), "head": lin(V, Wd) * 3, "final.norm": (1 + rnd(1, std=0.2)).reshape(())}
    for i, l in enumerate(cfg["layers"]):
        p, m, f = f"l{i}.mix.", l["mixer"], l["mlp"]
        W[f"l{i}.norm1"] = (1 + rnd(1, std=0.2)).reshape(())
        W[f"l{i}.rg1"], W[f"l{i}.rg1.b"] = lin(Wd, Wd) * 2, rnd(Wd, std=0.5)
        if l["type"] == "latent_attention":
            H, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            W[p + "dq"], W[p + "dq.norm"] = lin(m["q_rank"], Wd) * 2, 1 + rnd(m["q_rank"], std=0.2)
            W[p + "uq"] = lin(H * (d + r), m["q_rank"]) * 2
            W[p + "dkv"], W[p + "dkv.norm"] = lin(m["kv_rank"] + r, Wd) * 2, 1 + rnd(m["kv_rank"], std=0.2)
            W[p + "uk"], W[p + "uv"] = lin(H * d, m["kv_rank"]) * 2, lin(H * dv, m["kv_rank"]) * 2
            W[p + "g"], W[p + "o"] = lin(H * dv, Wd) * 2, lin(Wd, H * dv)
        elif l["type"] == "mlstm":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            W[p + "q"], W[p + "k"], W[p + "v"] = lin(H * d, Wd) * 2, lin(H * d, Wd) * 2, lin(H * dv, Wd) * 2
            W[p + "i"], W[p + "i.b"] = lin(H, Wd) * 3, rnd(H)
            W[p + "f"], W[p + "f.b"] = lin(H, Wd) * 3, rnd(H) + 2.0
            W[p + "g"], W[p + "norm"], W[p + "o"] = lin(H * dv, Wd) * 2, 1 + rnd(H * dv, std=0.2), lin(Wd, H * dv)
        else:
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[p + "q"], W[p + "q.norm"] = lin(H * d, Wd) * 2, 1 + rnd(d, std=0.3)
            W[p + "k"], W[p + "k.norm"] = lin(G * d, Wd) * 2, 1 + rnd(d, std=0.3)
            W[p + "v"], W[p + "sink"], W[p + "o"] = lin(G * dv, Wd) * 2, rnd(H), lin(Wd, H * dv)
        if f is None:
            continue
        p = f"l{i}.mlp."
        W[f"l{i}.norm2"] = (1 + rnd(1, std=0.2)).reshape(())
        W[f"l{i}.rg2"], W[f"l{i}.rg2.b"] = lin(Wd, Wd) * 2, rnd(Wd, std=0.5)
        if f["kind"] == "dense":
            W[p + "up"], W[p + "down"], W[p + "act"] = lin(f["ff"], Wd) * 2, lin(Wd, f["ff"]), rnd(4, std=0.7)
        else:
            n = f["router"]["experts"]
            W[p + "router"], W[p + "correction"] = lin(n, Wd) * 3, rnd(n, std=0.1)
            names = [f"e{e}." for e in range(n)] + (["shared."] if f.get("shared") else [])
            for e in names:
                ff = f["shared"]["ff"] if e == "shared." else f["expert"]["ff"]
                W[p + e + "gate"], W[p + e + "up"], W[p + e + "down"] = lin(ff, Wd) * 2, lin(ff, Wd) * 2, lin(Wd, ff)
    return {k: v.bfloat16().float() for k, v in W.items()}


def save_checkpoint(path, cfg, W):
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return path
