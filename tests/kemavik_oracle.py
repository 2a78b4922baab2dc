"""Plain whole-sequence implementation of the Kemavik design, used as the oracle of
``tests/test_kemavik.py``. One function per mechanism, float64, token by token where the
design is recurrent, no cache, no batching, and no code shared with ``hipserve``.

A model is (config dict as in ``config.json``, dict of tensors under the checkpoint's names).
"""
from __future__ import annotations

import math

import torch

DT = torch.float64


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def out_norm(y, w, eps):
    """The norm of a sublayer's output: weights stored around zero."""
    return rms(y, eps) * (1.0 + w)


# ------------------------------------------------------------------ linear attention with decays
def blends(h, W, pre):
    """The five inputs r, k, v, g, w: each between the token's row and the previous one's (zeros before
    the first)."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return {s: h + (before - h) * W[pre + "mu." + s] for s in "rkvgw"}


def decay(xw, W, pre):
    """exp(-exp(.)) of the bottleneck's output plus w0: one number in (0, 1) per key channel and token."""
    return torch.exp(-torch.exp(torch.tanh(xw @ W[pre + "w1"].T) @ W[pre + "w2"].T + W[pre + "w0"].reshape(-1)))


def wkv_recurrence(r, k, v, w, u):
    """r, k, v, w [n, H, d], u [H, d]. Per head with state S [key, value] from zero:
    o_t = sum_key r_t (S + u k_t v_t^T);  S <- w_t S + k_t v_t^T (w_t scales the key rows)."""
    n, H, d = r.shape
    S = torch.zeros(H, d, d, dtype=DT)
    o = torch.zeros(n, H, d, dtype=DT)
    for t in range(n):
        for hh in range(H):
            outer = torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = r[t, hh] @ (S[hh] + u[hh][:, None] * outer)
            S[hh] = w[t, hh][:, None] * S[hh] + outer
    return o


def wkv_mixer(h, m, W, pre, eps):
    n = h.shape[0]
    H, d = m["heads"], m["dim"]
    x = blends(h, W, pre)
    r, k, v = ((x[s] @ W[pre + s].T).view(n, H, d) for s in "rkv")
    gate = silu(x["g"] @ W[pre + "g"].T)
    w = decay(x["w"], W, pre).view(n, H, d)
    o = wkv_recurrence(r, k, v, w, W[pre + "u"].view(H, d))
    o = rms(o, eps).reshape(n, H * d) * W[pre + "norm"] * gate
    return o @ W[pre + "o"].T


# ------------------------------------------------------------------ differential attention
def causal_softmax_attention(q, k, v, scale):
    """q [n, d], k [n, d], v [n, dv]: row i over keys j <= i."""
    n = q.shape[0]
    s = (q @ k.T) * scale
    s = s.masked_fill(torch.triu(torch.ones(n, n, dtype=torch.bool), 1), -math.inf)
    return torch.softmax(s, -1) @ v


def lam_of(m, W, pre):
    return (torch.exp(W[pre + "lq1"] @ W[pre + "lk1"]) - torch.exp(W[pre + "lq2"] @ W[pre + "lk2"]) + m["diff"]).item()


def diff_keys_values(h, m, W, pre, eps):
    """What an attention layer with projections of its own leaves for layers that read its keys and values:
    keys [n, G, 2, d] after their norm, values [n, G, dv]."""
    n = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ W[pre + "k"].T + W[pre + "k.b"]).view(n, G, 2, d)
    k = rms(k, eps) * W[pre + "k.norm"]
    v = (h @ W[pre + "v"].T + W[pre + "v.b"]).view(n, G, dv)
    return k, v


def diff_attention_mixer(h, m, W, pre, eps, kv=None):
    """kv: (keys, values) of the layer named by ``kv_from``, or None for a layer with its own."""
    n = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[pre + "q"].T + W[pre + "q.b"]).view(n, H, 2, d)
    q = rms(q, eps) * W[pre + "q.norm"]
    k, v = kv if kv is not None else diff_keys_values(h, m, W, pre, eps)
    lam = lam_of(m, W, pre)
    out = torch.zeros(n, H, dv, dtype=DT)
    for hh in range(H):
        g = hh // (H // G)
        a1 = causal_softmax_attention(q[:, hh, 0], k[:, g, 0], v[:, g], m["scale"])
        a2 = causal_softmax_attention(q[:, hh, 1], k[:, g, 1], v[:, g], m["scale"])
        out[:, hh] = rms(a1 - lam * a2, eps) * (1.0 - m["diff"])
    return out.reshape(n, H * dv) @ W[pre + "o"].T + W[pre + "o.b"], (k, v)


# ------------------------------------------------------------------ feed-forwards
def dense_ff(h, W, pre):
    return torch.relu(h @ W[pre + "up"].T) ** 2 @ W[pre + "down"].T


def gated_ff(h, W, pre):
    return (silu(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def route(h, f, W, pre):
    """(chosen outputs [n, top], their weights): softmax over all router outputs; chosen by score +
    correction, weighted by the score itself times router.scale."""
    r = f["router"]
    s = torch.softmax(h @ W[pre + "router"].T, -1)
    idx = torch.topk(s + W[pre + "correction"], r["top"], -1).indices
    return idx, s.gather(1, idx) * r["scale"]


def moe_ff(h, f, W, pre):
    E = f["router"]["experts"]
    idx, wgt = route(h, f, W, pre)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(idx[t].tolist(), wgt[t]):
            out[t] += a * (h[t] if e >= E else gated_ff(h[t:t + 1], W, f"{pre}e{e}.")[0])   # identity experts: e >= E
    if f.get("shared"):
        out = out + gated_ff(h, W, pre + "shared.")
    return out


def feed_forward(h, f, W, pre):
    return dense_ff(h, W, pre) if f["kind"] == "dense" else moe_ff(h, f, W, pre)


# ------------------------------------------------------------------ the model
def forward(cfg: dict, tensors: dict, tokens, capture: list | None = None):
    """Logits [n, vocab] of one sequence; ``capture`` collects the stream after every layer."""
    W = {k: v.to(DT) for k, v in tensors.items() if v.is_floating_point()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens)]
    kept = {}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        if l["type"] == "wkv":
            y = wkv_mixer(x, m, W, p + "mix.", eps)
        else:
            src = m.get("kv_from")
            y, kept[i] = diff_attention_mixer(x, m, W, p + "mix.", eps, None if src is None else kept[src])
        x = x + out_norm(y, W[p + "norm1"], eps)
        if l["mlp"] is not None:
            x = x + out_norm(feed_forward(x, l["mlp"], W, p + "mlp."), W[p + "norm2"], eps)
        if capture is not None:
            capture.append(x.clone())
    return out_norm(x, W["final.norm"], eps) @ W["head"].T


# ------------------------------------------------------------------ small configs and random weights
def wkv_layer(heads=3, dim=8, mlp=None):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


def attn_layer(heads=4, kv_heads=2, dim=8, vdim=12, scale=None, diff=0.3, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5, "diff": diff}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=12, identity=2, scale=1.5, shared=20):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity, "scale": scale}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def make_config(layers, width=32, vocab=96, eps=1e-5):
    return {"architecture": "Kemavik", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}


def make_weights(cfg, seed=0, gain=1.0, rank=5):
    """Random checkpoint tensors (values representable in bf16) under the design's names."""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).bfloat16().float()

    def lin(o, i):
        return rnd(o, i, std=gain / math.sqrt(i))

    W = {"embed": rnd(V, Wd), "head": lin(V, Wd) * 3, "final.norm": rnd(Wd, std=0.1)}
    for i, l in enumerate(cfg["layers"]):
        p, m, f = f"l{i}.mix.", l["mixer"], l["mlp"]
        W[f"l{i}.norm1"] = rnd(Wd, std=0.1)
        if l["type"] == "wkv":
            N = m["heads"] * m["dim"]
            for s in "rkvgw":
                W[p + "mu." + s] = torch.rand(Wd, generator=g).bfloat16().float()
            for s in "rkvg":
                W[p + s] = lin(N, Wd) * 2
            W[p + "w1"], W[p + "w2"], W[p + "w0"] = lin(rank, Wd) * 2, rnd(N, rank, std=0.7), rnd(N) - 1.0
            W[p + "u"], W[p + "norm"], W[p + "o"] = rnd(m["heads"], m["dim"], std=0.5), 1 + rnd(N, std=0.2), lin(Wd, N)
        else:
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[p + "q"], W[p + "q.b"], W[p + "q.norm"] = lin(2 * H * d, Wd) * 2, rnd(2 * H * d, std=0.3), 1 + rnd(d, std=0.3)
            if m.get("kv_from") is None:
                W[p + "k"], W[p + "k.b"], W[p + "k.norm"] = lin(2 * G * d, Wd) * 2, rnd(2 * G * d, std=0.3), 1 + rnd(d, std=0.3)
                W[p + "v"], W[p + "v.b"] = lin(G * dv, Wd), rnd(G * dv, std=0.3)
            for s in ("lq1", "lk1", "lq2", "lk2"):
                W[p + s] = rnd(d, std=0.3)
            W[p + "o"], W[p + "o.b"] = lin(Wd, H * dv), rnd(Wd, std=0.2)
        if f is None:
            continue
        p = f"l{i}.mlp."
        W[f"l{i}.norm2"] = rnd(Wd, std=0.1)
        if f["kind"] == "dense":
            W[p + "up"], W[p + "down"] = lin(f["ff"], Wd) * 2, lin(Wd, f["ff"])
        else:
            r = f["router"]
            n = r["experts"] + r.get("identity", 0)
            W[p + "router"], W[p + "correction"] = lin(n, Wd) * 3, rnd(n, std=0.1)
            names = [f"e{e}." for e in range(r["experts"])] + (["shared."] if f.get("shared") else [])
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
