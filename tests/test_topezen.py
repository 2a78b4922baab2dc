"""The Topezen layer-list decoder against the plain oracle of tests/topezen_oracle.py: every
mechanism alone (whole rows, portions, one token from the cache / state), and the engine (paged
cache, state slots, batching, scheduler) against whole-sequence oracle logits: prefill vs
token-by-token decoding, prompt portions down to two tokens, unequal requests in one batch,
freed pages and slots used again, window edges and kept first tokens, far keys at page borders,
first tokens, long decoding, other sizes, greedy generation.
The same tests run on the CPU (reference ops) and, marked gpu, on the HIP kernels in bf16 and fp32."""
import math

import pytest
import torch

from hipserve.config import (DenseFFSpec, EngineConfig, LatentAttentionSpec, MLstmSpec, RoutedMoESpec, TopezenConfig,
                             WindowAttentionSpec)
from hipserve.engine.llm_engine import LLMEngine
from hipserve.engine.request import SamplingParams
from hipserve.engine.trace import TraceSession, build_engine
from hipserve.models.mixers import attach_side, make_ff, make_mixer
from hipserve.ops import get_ops
from hipserve.parallel.comm import TPGroup

from . import topezen_oracle as O
from .test_fikizen import CPU, TARGETS, TOL, check_all, one_seq_meta, portions, rel_err, replay, rows, tokens

EPS = 1e-5


def base_config(**kw):
    """Latent attention + dense, matrix memory + experts, window attention + experts, a matrix memory of other
    sizes without a feed-forward, latent attention + experts of other sizes, window attention + dense."""
    layers = [O.latent_layer(mlp=O.dense()), O.mlstm_layer(mlp=O.moe()), O.attn_layer(mlp=O.moe()),
              O.mlstm_layer(heads=3, dim=5, vdim=7, gate_cap=4.0),
              O.latent_layer(heads=2, dim=6, rot_dim=6, vdim=9, q_rank=7, kv_rank=11, base=500.0,
                             mlp=O.moe(experts=4, top=3, count=2, keep=2, shared=0)),
              O.attn_layer(heads=3, kv_heads=3, dim=6, vdim=5, softcap=3.0, size=6, keep_first=1, mlp=O.dense(ff=17))]
    return O.make_config(layers, **kw)


def session(tmp_path, cfg, W, target, max_tokens=512, name="m"):
    path = O.save_checkpoint(str(tmp_path / name), cfg, W)
    eng = build_engine(path, target[1], max_tokens, target[0])
    if target[0] == "cuda":  # the HIP kernels are the path that runs
        assert eng.runner.ops.name == "hip" and hasattr(eng.runner.ops._cell, "mlstm")   # loads the library
    return TraceSession(eng)


def d64(W, prefix="l0.mix."):
    return {k[len(prefix):]: v.double() for k, v in W.items() if k.startswith(prefix)}


# ---------------------------------------------------------------- mechanisms alone
def build_mixer(layer, W, target, width):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    spec = TopezenConfig.from_dict(O.make_config([layer], width=width)).layers[0].mixer
    mix = make_mixer(spec, width, EPS, dev, dt, get_ops(dev))
    if hasattr(mix.ops, "norm_library"):
        mix.ops.norm_library = "cell"
    mix.load(lambda k: W[k], "l0.mix.")
    return mix, dev, dt


def run_mixer(layer, W, h, target, cuts, width=24, slot=1, total=160):
    """The layer's mixer on rows h, cut into the given row ranges, each run from what the one before left in
    the cache / state (whose slot held garbage before the first)."""
    mix, dev, dt = build_mixer(layer, W, target, width)
    _, nblk = one_seq_meta(1, dev, total=total)
    cache = torch.zeros(nblk, 4, mix.cache_dim, device=dev, dtype=dt) if mix.cache_dim else None
    state = None
    if mix.state_shapes:
        state = [torch.full(s, 7.0, device=dev, dtype=torch.float32) for s in mix.state_shapes(3)]
    parts = []
    for a, b in cuts:
        meta, _ = one_seq_meta(b - a, dev, start=a, slot=slot, total=total)
        meta.max_ctx = b
        parts.append(mix.forward(h[a:b].to(dev, dt), meta, cache, state))
    return torch.cat(parts), state


CUTS = [[(0, 90)], [(0, 37), (37, 89), (89, 90)], [(0, 1), (1, 3), (3, 5), (5, 64), (64, 66), (66, 90)]]
LONG = [(0, 150), (150, 297), (297, 298), (298, 299), (299, 300)]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=1, dim=3, rot_dim=2, vdim=1, q_rank=1, kv_rank=2),
                                   dict(heads=5, dim=10, rot_dim=6, vdim=70, q_rank=9, kv_rank=20, scale=0.4, base=77.0),
                                   dict(heads=4, dim=32, rot_dim=16, vdim=24, q_rank=24, kv_rank=64)])
def test_latent_attention_alone(target, shape):
    l = O.latent_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=3)
    h = rows(90, 24, 1).double()
    want = O.latent_attention(h, d64(W), l["mixer"], EPS)
    for cuts in CUTS:
        assert rel_err(run_mixer(l, W, h.float(), target, cuts)[0], want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
def test_latent_attention_many_keys_and_what_matters(target):
    """Sizes the matrix-core kernel takes in bf16, with enough keys that a row decoded alone splits them into runs.
    The oracle shows what a wrong reading would change: the pairing of rotated coordinates, the rotation of the
    shared key part, the gate per channel."""
    l = O.latent_layer(heads=4, dim=32, rot_dim=32, vdim=16, q_rank=32, kv_rank=64, base=100.0)
    W = O.make_weights(O.make_config([l], width=24), seed=4)
    h = rows(300, 24, 2).double()
    w = d64(W)
    want = O.latent_attention(h, w, l["mixer"], EPS)
    half = dict(w)   # rotate-half pairing of the same weights
    idx = torch.cat([torch.arange(0, 32, 2), torch.arange(1, 32, 2)])
    half["dkv"] = torch.cat([w["dkv"][:64], w["dkv"][64:][idx.argsort()]])
    assert rel_err(O.latent_attention(h, half, l["mixer"], EPS), want) > 0.05
    flat = dict(w, g=torch.zeros_like(w["g"]))
    assert rel_err(O.latent_attention(h, flat, l["mixer"], EPS), want) > 0.05
    got, _ = run_mixer(l, W, h.float(), target, LONG, total=304)
    assert rel_err(got, want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=1, dim=1, vdim=1), dict(heads=5, dim=17, vdim=3, gate_cap=2.0),
                                   dict(heads=2, dim=64, vdim=40), dict(heads=1, dim=70, vdim=130, gate_cap=30.0),
                                   dict(heads=1, dim=300, vdim=20), dict(heads=1, dim=8, vdim=1100)])
def test_matrix_memory_alone(target, shape):
    l = O.mlstm_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=5)
    h = rows(90, 24, 3).double()
    want, st = O.mlstm(h, d64(W), l["mixer"], EPS)
    for cuts in CUTS:
        got, state = run_mixer(l, W, h.float(), target, cuts)
        assert rel_err(got, want) < TOL[target[1]]
        # the slot holds the state scaled by exp(-m): compare what does not depend on the path of m
        m = state[2][1].double().cpu()
        held = state[0][1].double().cpu() * torch.exp(m - st[2])[:, None, None]
        assert float((held - st[0]).norm() / st[0].norm()) < (2e-2 if target[1] == "bfloat16" else 1e-4)
        assert float(state[0][0].min()) == 7.0 and float(state[2][2].max()) == 7.0   # the other slots are untouched


@pytest.mark.parametrize("target", TARGETS)
def test_matrix_memory_gates_and_floor_matter(target):
    """Inputs on which a wrong reading shows: a forget gate far from 1 (decay), gates beyond the cap, an input gate
    so small that the maximum stays at its start 0 (not minus infinity) and the floor exp(-m) of the
    denominator decides; the product path follows on all of them."""
    l = O.mlstm_layer(heads=2, dim=8, vdim=6, gate_cap=3.0)
    W = O.make_weights(O.make_config([l], width=24), seed=6)
    W["l0.mix.i"] *= 6.0                       # |W_i h| well beyond the cap
    W["l0.mix.f.b"] = torch.tensor([-2.0, 6.0])
    W["l0.mix.i.b"] = torch.tensor([0.0, -9.0])   # head 1: i ~ -3 < f + 0, so m stays near 0 for a while
    h = rows(60, 24, 4).double()
    w = d64(W)
    want, _ = O.mlstm(h, w, l["mixer"], EPS)
    for change in (dict(gate_cap=1e6), ):
        assert rel_err(O.mlstm(h, w, dict(l["mixer"], **change), EPS)[0], want) > 0.03
    no_decay = dict(w)
    no_decay["f.b"] = torch.full_like(w["f.b"], 30.0)
    assert rel_err(O.mlstm(h, no_decay, dict(l["mixer"], gate_cap=100.0), EPS)[0], want) > 0.03
    for cuts in ([(0, 60)], [(0, 7), (7, 8), (8, 9), (9, 41), (41, 60)]):
        assert rel_err(run_mixer(l, W, h.float(), target, cuts)[0], want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
def test_matrix_memory_long_and_tiny_values(target):
    """300 tokens with gates that drive the running maximum far from 0 in both directions."""
    l = O.mlstm_layer(heads=2, dim=16, vdim=16, gate_cap=11.0)
    W = O.make_weights(O.make_config([l], width=24), seed=7)
    W["l0.mix.i.b"] = torch.tensor([8.0, -8.0])
    h = rows(300, 24, 5).double()
    want, _ = O.mlstm(h, d64(W), l["mixer"], EPS)
    got, _ = run_mixer(l, W, h.float(), target, [(0, 130), (130, 131), (131, 195), (195, 300)], total=304)
    # bf16: the rows as a whole (the worst single row of 300 lands on an output that is small all over)
    check_all({("s", p): r for p, r in enumerate(got.float().cpu())}, "s", want, TOL[target[1]])


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=1, kv_heads=1, dim=6, vdim=1, size=1, keep_first=1),
                                   dict(heads=6, kv_heads=2, dim=16, vdim=3, size=200, keep_first=0, softcap=2.0),
                                   dict(heads=36, kv_heads=2, size=5, keep_first=9),
                                   dict(heads=3, kv_heads=1, dim=80, vdim=130, size=33, keep_first=31),
                                   dict(heads=4, kv_heads=2, dim=32, vdim=64, size=48, keep_first=12, scale=0.3)])
def test_window_attention_alone(target, shape):
    l = O.attn_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=8)
    h = rows(90, 24, 6).double()
    want = O.sink_attention(h, d64(W), l["mixer"], EPS)
    for cuts in CUTS:
        assert rel_err(run_mixer(l, W, h.float(), target, cuts)[0], want) < TOL[target[1]]


def planted_attention(size, keep, n, seed, softcap=25.0):
    """A window-attention layer whose queries find keys through reversed weights: the key projection is the first
    head's query projection with its columns reversed, so a row scores highest against the key of the row that is
    its own reversed. Returns the layer, weights and a function placing a (key row, probe row) pair into rows."""
    l = O.attn_layer(heads=2, kv_heads=1, dim=24, vdim=8, scale=2.0, softcap=softcap, size=size, keep_first=keep)
    W = O.make_weights(O.make_config([l], width=24), seed=seed)
    W["l0.mix.k"] = W["l0.mix.q"][:24].flip(1).clone()
    W["l0.mix.k.norm"] = W["l0.mix.q.norm"].clone()
    return l, W


@pytest.mark.parametrize("target", TARGETS)
def test_window_edges_kept_first_tokens_cap_and_sink(target):
    """Probe rows whose key of interest sits just inside and just outside the window, on the last kept position and
    on the first one that is not kept, far behind the window; in prompt portions and in rows decoded alone, with
    pages of 4 tokens so every edge also meets a page border somewhere. The oracle shows that each of these keys,
    the cap and the sink change the probe's output."""
    size, keep, n = 36, 6, 300
    l, W = planted_attention(size, keep, n, 9)
    h = rows(n, 24, 7).double()
    pairs = [(100, 135), (100, 136), (5, 200), (6, 210), (0, 299), (262, 297), (263, 298), (150, 185), (150, 186)]
    for a, b in pairs:
        h[b] = h[a].flip(0) * 1.5
    w = d64(W)
    m = l["mixer"]
    want = O.sink_attention(h, w, m, EPS)
    seen = {(100, 135): True, (100, 136): False, (5, 200): True, (6, 210): False, (0, 299): True, (262, 297): True,
            (263, 298): True, (150, 185): True, (150, 186): False}
    for (a, b), vis in seen.items():
        other = h.clone()
        other[a] = rows(1, 24, 99)[0].double()
        moved = rel_err(O.sink_attention(other, w, m, EPS)[b:b + 1], want[b:b + 1])
        assert (moved > 0.05) == vis, (a, b, moved)
    assert rel_err(O.sink_attention(h, w, dict(m, softcap=1e6), EPS), want) > 0.02
    assert rel_err(O.sink_attention(h, dict(w, sink=w["sink"] - 30.0), m, EPS), want) > 0.02
    for cuts in ([(0, n)], [(0, 135), (135, 137), (137, 185), (185, 186), (186, 187), (187, 296)] + [(i, i + 1) for i in range(296, 300)],
                 [(0, 3), (3, 210), (210, 211), (211, 300)]):
        got, _ = run_mixer(l, W, h.float(), target, cuts, total=304)
        assert rel_err(got, want) < TOL[target[1]] * (1 if target[1] == "float32" else 2)


def build_ff(f, W, target, width, side=False):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    cfg = O.make_config([O.mlstm_layer(mlp=f)], width=width)
    spec = TopezenConfig.from_dict(cfg).layers[0].mlp
    ops = get_ops(dev)
    if hasattr(ops, "norm_library"):
        ops.norm_library = "cell"
    ff = make_ff(spec, width, dev, dt, ops, EPS)
    ff.load(lambda k: W[k], "l0.mlp.")
    if side:
        attach_side(ff, W["l0.rg2"])
    return ff, ops, dev, dt


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("ff", [40, 1, 333, 5000])
def test_polynorm_feed_forward_alone(target, ff):
    f = O.dense(ff=ff)
    W = O.make_weights(O.make_config([O.mlstm_layer(mlp=f)], width=24), seed=10)
    h = rows(50, 24, 8)
    want = O.polynorm_ff(h.double(), d64(W, "l0.mlp."), EPS)
    for side in (False, True):
        mod, _, dev, dt = build_ff(f, W, target, 24, side)
        assert rel_err(mod.forward(h.to(dev, dt)), want) < TOL[target[1]]
        assert (mod.side_out is not None) == side
    w = d64(W, "l0.mlp.")
    assert rel_err(O.polynorm_ff(h.double(), dict(w, act=w["act"] * torch.tensor([1.0, 0.0, 1.0, 1.0])), EPS), want) > 0.02


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(experts=1, top=1, count=1, keep=1, shared=0), dict(experts=8, top=4, count=4, keep=2),
                                   dict(experts=12, top=3, count=2, keep=1, ff=7, shared=5), dict(experts=9, top=9, count=3, keep=3),
                                   dict(experts=70, top=5, count=10, keep=3, ff=4)])
def test_routed_experts_alone(target, shape):
    """Choice and weights of the router, and the mixture's output through the gated block update. The corrections are
    large and negative for some experts, so choice scores go below zero: a masked group must count as minus infinity."""
    f = O.moe(**shape)
    W = O.make_weights(O.make_config([O.mlstm_layer(mlp=f)], width=24), seed=11)
    n = f["router"]["experts"]
    W["l0.mlp.correction"] = (torch.randn(n, generator=torch.Generator().manual_seed(1)) * 0.5 - 0.6).bfloat16().float()
    h = rows(70, 24, 9)
    w = d64(W, "l0.mlp.")
    ids_want, ws_want = O.route(h.bfloat16().double() if target[1] == "bfloat16" else h.double(), w, f["router"])
    mod, ops, dev, dt = build_ff(f, W, target, 24, side=True)
    ye, pair_slot, ids, wts, _, _, shared = mod.forward(h.to(dev, dt))
    order = ids.long().cpu().sort(-1)
    assert torch.equal(order.values, ids_want.sort(-1).values)
    got_w = wts.cpu().double().gather(1, order.indices)
    assert torch.allclose(got_w, ws_want.gather(1, ids_want.sort(-1).indices), atol=1e-5 if target[1] == "float32" else 2e-2)
    assert torch.allclose(wts.sum(-1).cpu(), torch.ones(70), atol=1e-5)
    # the mixture's output, gated, summed into a stream of zeros
    residual = torch.zeros(70, 24, device=dev)
    h1 = torch.empty(70, 24, device=dev, dtype=dt)
    b2 = W["l0.rg2.b"].to(dev)
    one = torch.ones(1, device=dev)
    ops.gated_add_norms(h1, None, residual, one, None, EPS, None, ((ye, pair_slot, wts, shared), mod.side_out, b2))
    hd = h.double()
    want = O.moe_ff(hd, w, f) * O.sigmoid(O.lin(W["l0.rg2"].double(), hd) + W["l0.rg2.b"].double())
    assert rel_err(residual, want) < TOL[target[1]]
    assert rel_err(h1, O.rms_unit(want, EPS)) < TOL[target[1]]


def test_group_limit_changes_the_choice():
    f = O.moe(experts=8, top=2, count=4, keep=1)
    W = O.make_weights(O.make_config([O.mlstm_layer(mlp=f)], width=24), seed=12)
    h = rows(40, 24, 10).double()
    w = d64(W, "l0.mlp.")
    ids, _ = O.route(h, w, f["router"])
    assert bool(((ids // 2) == (ids // 2)[:, :1]).all())   # both chosen experts from one group of two
    free, _ = O.route(h, w, dict(f["router"], groups={"count": 1, "keep": 1}))
    assert not torch.equal(ids.sort(-1).values, free.sort(-1).values)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("width", [24, 3000])
def test_gated_block_update_alone(target, width):
    """Both sublayers' results gated and summed into the stream, both next norms from one mean square; weights of
    one number or one per channel; gates read from column slices of wider rows."""
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    ops = get_ops(dev)
    T = 9
    g = torch.Generator().manual_seed(13)
    r0, y1, y2 = (torch.randn(T, width, generator=g) for _ in range(3))
    wide1, wide2 = torch.randn(T, width + 5, generator=g), torch.randn(T, 2 * width, generator=g)
    b1, b2 = torch.randn(width, generator=g), torch.randn(width, generator=g)
    w1, w2 = torch.tensor([1.3]), torch.randn(width, generator=g)
    y1, y2, wide1, wide2 = (t.to(dt).float() for t in (y1, y2, wide1, wide2))
    want = r0.double() + torch.sigmoid(wide1[:, 5:].double() + b1) * y1 + torch.sigmoid(wide2[:, :width].double() + b2) * y2
    residual = r0.clone().to(dev)
    o1, o2 = torch.empty(T, width, device=dev, dtype=dt), torch.empty(T, width, device=dev, dtype=dt)
    ops.gated_add_norms(o1, o2, residual, w1.to(dev), w2.to(dev), EPS, (y1.to(dev, dt), wide1.to(dev, dt)[:, 5:], b1.to(dev)),
                        (y2.to(dev, dt), wide2.to(dev, dt)[:, :width], b2.to(dev)))
    assert torch.allclose(residual.cpu().double(), want, atol=1e-5)
    tol = TOL[target[1]]
    assert rel_err(o1, O.rms_unit(want, EPS) * 1.3) < tol and rel_err(o2, O.rms_unit(want, EPS) * w2.double()) < tol
    # no addend at all: only the norms; one addend only
    before = residual.clone()
    ops.gated_add_norms(o1, None, residual, w2.to(dev), None, EPS)
    assert torch.equal(residual, before) and rel_err(o1, O.rms_unit(want, EPS) * w2.double()) < tol
    ops.gated_add_norms(o1, None, residual, w1.to(dev), None, EPS, (y1.to(dev, dt), wide1.to(dev, dt)[:, 5:], b1.to(dev)))
    want = want + torch.sigmoid(wide1[:, 5:].double() + b1) * y1
    assert torch.allclose(residual.cpu().double(), want, atol=1e-5)


# ---------------------------------------------------------------- engine
@pytest.mark.parametrize("target", TARGETS)
def test_prefill_and_long_decoding(tmp_path, target):
    cfg = base_config()
    W = O.make_weights(cfg, seed=21)
    toks = tokens(70, cfg["vocab"], 1)
    ref, streams, _ = O.forward(cfg, W, toks, return_layers=True)
    sess = session(tmp_path, cfg, W, target)
    model = sess.engine.runner.model
    model.capture = []
    check_all(replay(sess, portions(toks, [len(toks)])), "a", ref, TOL[target[1]])   # the whole prompt at once
    for got, want in zip(model.capture, streams):                                    # the stream after every layer
        check_all({("s", p): r for p, r in enumerate(got)}, "s", want, TOL[target[1]])
    assert len(model.capture) == len(streams) == 6
    model.capture = None
    check_all(replay(sess, portions(toks, [10])), "a", ref, TOL[target[1]])          # 60 tokens one by one
    check_all(replay(sess, portions(toks, [1])), "a", ref, TOL[target[1]])           # from the very first token


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("sizes", [[2] * 40, [3, 2, 17, 2, 5, 31, 2], [16, 16, 16, 16], [33, 2, 2, 2]])
def test_portions(tmp_path, target, sizes):
    cfg = base_config()
    W = O.make_weights(cfg, seed=22)
    toks = tokens(83, cfg["vocab"], 2)
    ref = O.forward(cfg, W, toks)
    check_all(replay(session(tmp_path, cfg, W, target), portions(toks, sizes)), "a", ref, TOL[target[1]])


@pytest.mark.parametrize("target", TARGETS)
def test_unequal_requests_in_one_batch_and_reuse(tmp_path, target):
    """Up to four live requests of unequal length, portions beside single tokens; finished requests
    give pages and slots back and later ones take them; the pool is small enough that they must."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=23)
    V = cfg["vocab"]
    reqs = {f"r{k}": tokens(n, V, 20 + k) for k, n in enumerate([61, 1, 23, 40, 2, 35, 50, 18])}
    refs = {k: O.forward(cfg, W, t) for k, t in reqs.items()}
    sess = session(tmp_path, cfg, W, target, max_tokens=64 * 4)
    order = list(reqs)
    live, at, steps, cuts = [], {}, [], [5, 1, 2, 9, 1, 1, 3, 16, 1, 2]
    n = 0
    while order or live:
        while order and len(live) < 4:
            live.append(order.pop(0))
        step = []
        for j, rid in enumerate(list(live)):
            if (n + j) % 5 == 4 and len(live) > 1:
                continue  # a request may be left out of a step
            a = at.get(rid, 0)
            c = min(cuts[(n + 3 * j) % len(cuts)], len(reqs[rid]) - a)
            end = a + c == len(reqs[rid])
            step.append((rid, reqs[rid][a:a + c], list(range(c)), end))
            at[rid] = a + c
            if end:
                live.remove(rid)
        if step:
            steps.append(step)
        n += 1
    got = replay(sess, steps)
    for rid, ref in refs.items():
        check_all(got, rid, ref, TOL[target[1]])
    assert sess.engine.blocks.num_free() == sess.engine.blocks.num_blocks
    assert sess.engine.states.num_free() == 4


def planted_model(far, probes, n, seed):
    """A model whose first layer is latent attention that finds keys by content: one head, no rotated part worth
    mentioning, a key up-projection equal to the query's and a key latent made from the query latent's weights with
    the columns reversed, so a probe token whose embedding is a far token's reversed scores highest against it (and
    not against itself); a window attention layer follows."""
    lay = [O.latent_layer(heads=1, dim=16, rot_dim=2, vdim=8, q_rank=16, kv_rank=16, scale=1.5, mlp=O.dense(24)),
           O.attn_layer(heads=2, kv_heads=1, dim=24, vdim=8, scale=1.0, softcap=30.0, size=20, keep_first=2, mlp=O.moe())]
    cfg = O.make_config(lay, width=32, vocab=100 + 2 * len(far), scale=2.0)
    W = O.make_weights(cfg, seed=seed)
    p = "l0.mix."
    W[p + "dkv"][:16] = W[p + "dq"].flip(1).clone()
    W[p + "dkv.norm"] = W[p + "dq.norm"].clone()
    W[p + "uk"] = W[p + "uq"][:16].clone()
    toks = [t % 100 for t in tokens(n, 1000, seed)]
    for i, (a, b) in enumerate(zip(far, probes)):
        W["embed"][101 + 2 * i] = W["embed"][100 + 2 * i].flip(0).clone()
        toks[a], toks[b] = 100 + 2 * i, 101 + 2 * i   # token ids used nowhere else
    return cfg, W, toks


@pytest.mark.parametrize("target", TARGETS)
def test_far_keys_at_page_borders(tmp_path, target):
    """Keys hundreds of tokens back, in the last and the first slot of a page (the replay engine's pages hold
    16 tokens) and at the very first position, asked for from inside a prompt and by tokens decoded alone.
    Changing the far token moves the probe's logits, so a lost or misplaced key shows."""
    far, probes = [0, 47, 48, 175], [300, 317, 322, 325]
    cfg, W, toks = planted_model(far, probes, 330, 27)
    ref = O.forward(cfg, W, toks)
    for a, b in zip(far, probes):
        other = list(toks)
        other[a] = 7
        assert rel_err(O.forward(cfg, W, other)[b:b + 1], ref[b:b + 1]) > 0.05
    sess = session(tmp_path, cfg, W, target)
    tol = TOL[target[1]] * (1 if target[1] == "float32" else 2)
    check_all(replay(sess, portions(toks, [330])), "a", ref, tol)
    check_all(replay(sess, portions(toks, [129, 64, 107, 2, 18, 2])), "a", ref, tol)   # 300, 322, 325 in portions; 317 alone
    check_all(replay(sess, portions(toks, [299])), "a", ref, tol)                      # every probe decoded alone


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("variant", ["ones", "no_mlp", "memory_only", "attention_only", "wide", "odd", "equal"])
def test_other_sizes(tmp_path, target, variant):
    d = O.dense(ff=8)
    if variant == "ones":           # everything 1 that can be
        one = O.moe(experts=1, top=1, count=1, keep=1, shared=0)
        layers = [O.attn_layer(heads=1, kv_heads=1, dim=8, vdim=8, size=1, keep_first=0, mlp=one),
                  O.mlstm_layer(heads=1, dim=8, vdim=8, mlp=d),
                  O.latent_layer(heads=1, dim=8, rot_dim=2, vdim=8, q_rank=1, kv_rank=1, mlp=one)]
        cfg = O.make_config(layers, width=16, vocab=50, scale=1.0)
    elif variant == "no_mlp":
        layers = [O.mlstm_layer(), O.attn_layer(heads=7, kv_heads=7, dim=4, vdim=20), O.latent_layer(), O.mlstm_layer(heads=4, dim=3)]
        cfg = O.make_config(layers, width=48)
    elif variant == "memory_only":  # no paged cache at all
        layers = [O.mlstm_layer(mlp=d), O.mlstm_layer(heads=3, dim=4, vdim=4, mlp=O.moe())]
        cfg = O.make_config(layers, width=20)
    elif variant == "attention_only":  # no state slots at all; a window longer than the prompt, every token kept
        layers = [O.attn_layer(size=500, keep_first=0, mlp=d), O.latent_layer(mlp=O.moe()), O.attn_layer(size=2, keep_first=500)]
        cfg = O.make_config(layers, width=20)
    elif variant == "wide":         # head sizes that are no multiples of 8, 16 or 64, value heads wider than key heads
        layers = [O.attn_layer(heads=2, kv_heads=1, dim=72, vdim=136, mlp=O.dense(ff=70)), O.mlstm_layer(heads=2, dim=66, vdim=140),
                  O.latent_layer(heads=2, dim=20, rot_dim=10, vdim=7, q_rank=50, kv_rank=72, mlp=O.moe(experts=3, ff=65, count=1, keep=1, shared=9))]
        cfg = O.make_config(layers, width=24)
    elif variant == "odd":          # nothing a multiple of 4
        layers = [O.mlstm_layer(heads=3, dim=5, vdim=7, mlp=O.moe(experts=3, top=2, count=3, keep=2, ff=7, shared=5)),
                  O.attn_layer(heads=3, kv_heads=1, dim=6, vdim=5, size=7, keep_first=3, mlp=O.dense(ff=11)),
                  O.latent_layer(heads=3, dim=5, rot_dim=6, vdim=7, q_rank=9, kv_rank=11)]
        cfg = O.make_config(layers, width=30, vocab=53)
    else:                           # sizes that a model may happen to make equal: every head size and rank the same
        layers = [O.latent_layer(heads=2, dim=16, rot_dim=16, vdim=16, q_rank=16, kv_rank=16, mlp=O.dense(ff=32)),
                  O.mlstm_layer(heads=2, dim=16, vdim=16, mlp=O.moe(experts=4, top=2, count=2, keep=2, ff=16, shared=16)),
                  O.attn_layer(heads=2, kv_heads=2, dim=16, vdim=16, size=16, keep_first=16, mlp=O.dense(ff=32))]
        cfg = O.make_config(layers, width=32, vocab=77, eps=1e-3)
    W = O.make_weights(cfg, seed=27)
    toks = tokens(45, cfg["vocab"], 5)
    ref = O.forward(cfg, W, toks)
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [45])), "a", ref, TOL[target[1]])
    check_all(replay(sess, portions(toks, [4, 9, 2, 13])), "a", ref, TOL[target[1]])


def test_config_reader():
    cfg = base_config(eps=3e-4, scale=7.5)
    c = TopezenConfig.from_dict(cfg)
    assert c.norm_eps == 3e-4 and c.embed_scale == 7.5 and c.num_layers == 6 and [r[0] for r in c.runs()] == list(range(6))
    la, ml, at = c.layers[0].mixer, c.layers[1].mixer, c.layers[2].mixer
    assert isinstance(la, LatentAttentionSpec) and (la.interleaved, la.gate, la.window, la.gate_size) == (True, "channel", 0, 18)
    assert (la.heads, la.dim, la.rot_dim, la.vdim, la.q_rank, la.kv_rank, la.rot_dims, la.key_dim) == (3, 8, 4, 6, 10, 12, 4, 16)
    assert isinstance(ml, MLstmSpec) and (ml.heads, ml.dim, ml.vdim, ml.gate_cap, ml.out_size) == (2, 8, 12, 10.0, 24)
    assert isinstance(at, WindowAttentionSpec) and (at.head_norm, at.sink, at.sink_weights, at.gate, at.bias, at.maps) == (True, True, True, False, False, 1)
    assert (at.window, at.keep_first, at.softcap, at.rot_dims, at.cache_dim) == (11, 3, 15.0, 0, 2 * 8 + 2 * 12)
    d, f = c.layers[0].mlp, c.layers[1].mlp
    assert isinstance(d, DenseFFSpec) and (d.ff, d.act) == (40, "polynorm")
    assert isinstance(f, RoutedMoESpec) and (f.experts, f.top, f.ff, f.shared_ff, f.groups, f.keep_groups, f.renorm, f.identity) == (6, 2, 12, 20, 3, 2, True, 0)
    assert c.layers[3].mlp is None and c.layers[4].mlp.shared_ff == 0
    bad = base_config()
    bad["layers"][1]["mlp"]["router"]["groups"]["count"] = 4   # six experts in four groups
    with pytest.raises(ValueError):
        TopezenConfig.from_dict(bad)
    bad = base_config()
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(NotImplementedError):
        TopezenConfig.from_dict(bad)


def assert_greedy(cfg, W, prompt, out, slack, flips=0):
    """Every generated token is an argmax (within ``slack``) of the oracle's logits over the tokens before it. In
    bf16 up to ``flips`` positions may differ: among a hundred routed tokens of a tiny random model some have two
    experts whose choice scores differ by 1e-4, which the rounding of the router's input decides the other way,
    and another expert moves the logits by far more than rounding does. The tokens after it are checked against
    the oracle on the engine's own continuation, so a lost state or key would still show on all of them."""
    lg = O.forward(cfg, W, prompt + out)
    bad = [(k, t, int(lg[len(prompt) + k - 1].argmax())) for k, t in enumerate(out)
           if lg[len(prompt) + k - 1][t] < lg[len(prompt) + k - 1].max() - slack]
    assert len(bad) <= flips, bad


@pytest.mark.parametrize("target", TARGETS)
def test_greedy_generation_through_the_scheduler(tmp_path, target):
    """LLMEngine.generate: the scheduler's own chunked prefill (a 24-token budget), batching of three
    prompts of unequal length and the sampler; every generated token is an argmax of the oracle's
    logits over the tokens before it."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=28)
    path = O.save_checkpoint(str(tmp_path / "g"), cfg, W)
    dev = target[0]
    ecfg = EngineConfig(model=path, dtype=target[1], device=dev, max_num_seqs=4, max_num_batched_tokens=24,
                        num_kv_blocks=64, max_model_len=256, enforce_eager=True)
    eng = LLMEngine(ecfg, tp=TPGroup(0, 1, None, torch.device("cuda", 0)) if dev == "cuda" else TPGroup())
    assert eng.states is not None and not eng.blocks.prefix_caching
    prompts = [tokens(n, cfg["vocab"], 30 + n) for n in (50, 3, 29)]
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True))
    # the GPU sampler holds a logits row as bf16 (steps of 1/32 between 4 and 8), whatever the model's dtype
    slack = 1e-3 if target == CPU else (0.07 if target[1] == "float32" else 0.15)
    for p, (out, _text, reason) in zip(prompts, res):
        assert len(out) == 12 and reason == "length"
        assert_greedy(cfg, W, p, out, slack, flips=1 if target[1] == "bfloat16" else 0)
    assert eng.states.num_free() == 4 and eng.blocks.num_free() == eng.blocks.num_blocks


@pytest.mark.gpu
def test_graph_decode_matches_eager_gpu(tmp_path):
    """Decode-only steps replay a captured hipGraph (state slots and block tables staged per step): same
    greedy tokens as the eager engine, and argmaxes of the oracle."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=29)
    path = O.save_checkpoint(str(tmp_path / "gd"), cfg, W)
    prompts = [tokens(n, cfg["vocab"], 40 + n) for n in (37, 5, 21, 2, 30)]
    sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    outs = []
    for eager in (True, False):
        ecfg = EngineConfig(model=path, dtype="bfloat16", device="cuda", max_num_seqs=4, max_num_batched_tokens=64,
                            num_kv_blocks=64, max_model_len=128, enforce_eager=eager)
        eng = LLMEngine(ecfg, tp=TPGroup(0, 1, None, torch.device("cuda", 0)))
        assert eng.runner.use_graphs != eager
        outs.append([r[0] for r in eng.generate(prompts, sp)])
        if not eager:
            assert eng.runner.stats["graph_steps"] > 0
    for p, out in zip(prompts, outs[1]):
        assert_greedy(cfg, W, p, out, 0.3, flips=2)
    same = sum(a == b for a, b in zip(outs[0], outs[1]))
    assert same >= len(prompts) - 1, (outs[0], outs[1])  # bf16 near-ties may flip one continuation


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_of_real_layers_gpu(tmp_path, dtype):
    """Head sizes and ranks of real models (in bf16 the matrix-core attention kernels and the packed expert path's
    shapes), prompts long enough that decode rows split their keys, against the CPU reference ops on the same
    checkpoint (the oracle's loops would take minutes at this size)."""
    lay = [O.latent_layer(heads=4, dim=64, rot_dim=32, vdim=64, q_rank=96, kv_rank=128, mlp=O.dense(ff=512)),
           O.mlstm_layer(heads=4, dim=64, vdim=128, gate_cap=15.0, mlp=O.moe(experts=8, top=2, ff=128, count=4, keep=2, shared=256)),
           O.attn_layer(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.125, softcap=50.0, size=160, keep_first=16,
                        mlp=O.moe(experts=8, top=2, ff=128, count=4, keep=2, shared=256))]
    cfg = O.make_config(lay, width=256, vocab=300, scale=16.0)
    W = O.make_weights(cfg, seed=31)
    toks = tokens(420, 300, 9)
    steps = portions(toks, [200, 190, 2])
    want = replay(session(tmp_path, cfg, W, CPU, name="c"), steps)
    got = replay(session(tmp_path, cfg, W, ("cuda", dtype), name="g"), steps)
    ref = torch.stack([torch.as_tensor(want[("a", p)]) for p in range(420)])
    check_all(got, "a", ref, TOL[dtype] * (5 if dtype == "float32" else 1))


def test_preset_and_cli_model_resolution(tmp_path):
    from hipserve.config import resolve_model_config
    from hipserve.models.registry import model_class

    cfg = base_config()
    path = O.save_checkpoint(str(tmp_path / "c"), cfg, O.make_weights(cfg, seed=1))
    m = resolve_model_config(path)
    assert isinstance(m, TopezenConfig) and model_class(m).__name__ == "TopezenModel"
    t = resolve_model_config("tiny-topezen")
    assert isinstance(t, TopezenConfig) and t.layers[3].mlp is None and t.layers[2].mixer.keep_first == 5


def random_config(seed):
    """A model of the design with sizes, head counts, layer order, windows and constants drawn at random, in the
    range of small real layers (multiples of 8 mostly, so that bf16 meets the matrix-core kernels too)."""
    g = torch.Generator().manual_seed(1000 + seed)

    def pick(*xs):
        return xs[int(torch.randint(0, len(xs), (1,), generator=g))]

    def feed_forward():
        kind = pick("dense", "moe", "moe", None)
        if kind == "dense":
            return O.dense(ff=pick(48, 96, 200))
        if kind == "moe":
            count = pick(1, 2, 4)
            per = pick(1, 2, 4)
            keep = pick(*range(1, count + 1))
            top = pick(*range(1, min(keep * per, 4) + 1))
            return O.moe(experts=count * per, top=top, ff=pick(16, 40), count=count, keep=keep, shared=pick(0, 24, 64))
        return None

    layers = []
    for _ in range(pick(3, 4, 5)):
        kind = pick("latent", "mlstm", "attention")
        if kind == "latent":
            rot = pick(8, 16, 32)
            layers.append(O.latent_layer(heads=pick(1, 2, 4, 5), dim=pick(8, 16, 32), rot_dim=rot, vdim=pick(8, 24, 32),
                                         q_rank=pick(16, 40, 64), kv_rank=pick(32, 64), base=pick(1e2, 1e4, 5e5),
                                         mlp=feed_forward()))
        elif kind == "mlstm":
            layers.append(O.mlstm_layer(heads=pick(1, 2, 4), dim=pick(8, 16, 32, 64), vdim=pick(8, 16, 48), gate_cap=pick(5.0, 15.0),
                                        mlp=feed_forward()))
        else:
            kv = pick(1, 2)
            layers.append(O.attn_layer(heads=kv * pick(1, 2, 4), kv_heads=kv, dim=pick(16, 32, 64), vdim=pick(16, 32, 40),
                                       softcap=pick(10.0, 30.0), size=pick(7, 16, 33, 64), keep_first=pick(0, 1, 8, 20),
                                       mlp=feed_forward()))
    return O.make_config(layers, width=pick(48, 64, 96), vocab=pick(60, 130), eps=pick(1e-6, 1e-5, 1e-4), scale=pick(1.0, 8.0))


def check_rows(got, rid, ref, dtype):
    """fp32: every row, as ``check_all``. bf16: 95 % of the rows within half the tolerance and at most two rows (or
    2 %) far off: a row whose two best experts' choice scores differ by 1e-4 is routed the other way after bf16
    rounding of the router's input and then differs as a whole, alone; a wrong key, state or window moves every row
    after it."""
    if dtype != "bfloat16":
        return check_all(got, rid, ref, TOL[dtype])
    n = ref.shape[0]
    g = torch.stack([torch.as_tensor(got[(rid, p)]) for p in range(n)]).float().cpu()
    r = torch.as_tensor(ref).float()
    d = (g - r) - (g - r).mean(-1, keepdim=True)
    w = r - r.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()
    assert float(torch.quantile(e, 0.95)) < TOL[dtype] / 2 and int((e > 3 * TOL[dtype]).sum()) <= max(2, n // 50), e


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("seed", range(6))
def test_random_configurations(tmp_path, target, seed):
    """Two requests of a randomly drawn model, one in portions beside the other's single tokens, after a whole-prompt
    run of the first; pages and slots of the first run are used again."""
    cfg = random_config(seed)
    W = O.make_weights(cfg, seed=50 + seed)
    a, b = tokens(150, cfg["vocab"], 60 + seed), tokens(70, cfg["vocab"], 80 + seed)
    ref_a, ref_b = O.forward(cfg, W, a), O.forward(cfg, W, b)
    sess = session(tmp_path, cfg, W, target, max_tokens=256)
    check_rows(replay(sess, portions(a, [150], rid="w")), "w", ref_a, target[1])
    steps, pa, pb = [], 0, 0
    cuts = [37, 2, 64, 1, 1, 30, 9, 1, 1, 1, 1, 1]
    while pa < len(a) or pb < len(b):
        step = []
        if pa < len(a):
            n = min(cuts[len(steps) % len(cuts)], len(a) - pa)
            step.append(("a", a[pa:pa + n], list(range(n)), pa + n == len(a)))
            pa += n
        if pb < len(b):
            n = 20 if pb == 0 else 1
            step.append(("b", b[pb:pb + n], list(range(n)), pb + n == len(b)))
            pb += n
        steps.append(step)
    got = replay(sess, steps)
    check_rows(got, "a", ref_a, target[1])
    check_rows(got, "b", ref_b, target[1])
