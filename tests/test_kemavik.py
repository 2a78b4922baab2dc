"""The Kemavik layer-list decoder against the plain oracle of tests/kemavik_oracle.py: every
mechanism alone (whole rows, portions, one token from the cache / state), and the engine (paged
cache, state slots, batching, scheduler) against whole-sequence oracle logits: prefill vs
token-by-token decoding, prompt portions down to two tokens, unequal requests in one batch,
freed pages and slots used again, far keys at page borders, first tokens, long decoding, other
sizes, layers that read another layer's keys and values, greedy generation.
The same tests run on the CPU (reference ops) and, marked gpu, on the HIP kernels in bf16 and fp32."""
import pytest
import torch

from hipserve.config import EngineConfig, KemavikConfig, RoutedMoESpec, WindowAttentionSpec, WkvSpec
from hipserve.engine.llm_engine import LLMEngine
from hipserve.engine.request import SamplingParams
from hipserve.engine.trace import TraceSession, build_engine
from hipserve.models.mixers import make_ff, make_mixer
from hipserve.ops import get_ops
from hipserve.parallel.comm import TPGroup

from . import kemavik_oracle as O
from .test_fikizen import CPU, TARGETS, TOL, check_all, one_seq_meta, portions, rel_err, replay, rows, tokens

EPS = 1e-5


def base_config(**kw):
    """Linear attention, attention + experts, a reader of its keys and values, another attention of other
    sizes with a reader two layers on, a layer without a feed-forward."""
    d, m = O.dense(), O.moe()
    layers = [O.wkv_layer(mlp=d), O.attn_layer(mlp=m), O.attn_layer(kv_from=1, mlp=d),
              O.attn_layer(heads=6, kv_heads=3, dim=4, vdim=5, diff=0.55, mlp=O.moe(experts=3, top=3, identity=1, shared=0)),
              O.wkv_layer(heads=2, dim=5), O.attn_layer(heads=3, kv_heads=3, dim=4, vdim=5, diff=0.1, kv_from=3, mlp=d)]
    return O.make_config(layers, **kw)


def session(tmp_path, cfg, W, target, max_tokens=512, name="m"):
    path = O.save_checkpoint(str(tmp_path / name), cfg, W)
    eng = build_engine(path, target[1], max_tokens, target[0])
    if target[0] == "cuda":  # the HIP kernels are the path that runs
        assert eng.runner.ops.name == "hip" and hasattr(torch.ops.hipserve_delta, "wkv")
    return TraceSession(eng)


def d64(W):
    return {k: v.double() for k, v in W.items()}


# ---------------------------------------------------------------- mechanisms alone
def build_mixers(layers, W, target, width):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    specs = [l.mixer for l in KemavikConfig.from_dict(O.make_config(layers, width=width)).layers]
    mixers = []
    for i, sp in enumerate(specs):
        mixers.append(make_mixer(sp, width, EPS, dev, dt, get_ops(dev)))
        mixers[-1].load(lambda k: W[k], f"l{i}.mix.")
    return mixers, dev, dt


def run_mixer(layer, W, h, target, cuts, width=24, slot=1):
    """The layer's mixer on rows h, cut into the given row ranges, each run from what the one before left in
    the cache / state (whose slot held garbage before the first)."""
    (mix,), dev, dt = build_mixers([layer], W, target, width)
    _, nblk = one_seq_meta(1, dev)
    cache = torch.zeros(nblk, 4, mix.cache_dim, device=dev, dtype=dt) if mix.cache_dim else None
    state = None
    if mix.state_shapes:
        state = [torch.full(s, 7.0, device=dev, dtype=torch.float32) for s in mix.state_shapes(3)]
    parts = []
    for a, b in cuts:
        meta, _ = one_seq_meta(b - a, dev, start=a, slot=slot)
        x = h[a:b].to(dev, torch.float32 if getattr(mix, "input32", False) else dt)
        parts.append(mix.forward(x, meta, cache, state))
    return torch.cat(parts)


CUTS = [[(0, 90)], [(0, 37), (37, 89), (89, 90)], [(0, 1), (1, 3), (3, 5), (5, 64), (64, 66), (66, 90)]]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=1, dim=4), dict(heads=5, dim=17), dict(heads=2, dim=64),
                                   dict(heads=1, dim=70)])
def test_linear_attention_alone(target, shape):
    l = O.wkv_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=3)
    h = rows(90, 24, 1).double()
    want = O.wkv_mixer(h, l["mixer"], d64(W), "l0.mix.", EPS)
    for cuts in CUTS:
        assert rel_err(run_mixer(l, W, h.float(), target, cuts), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
def test_bonus_decay_and_blends_matter(target):
    """The parts of the recurrence a wrong reading would drop: the current token's bonus, the decay (a state
    that never fades), the blend with the previous row (all blend weights zero)."""
    l = O.wkv_layer()
    W = O.make_weights(O.make_config([l], width=24), seed=4)
    h = rows(40, 24, 2).double()
    want = O.wkv_mixer(h, l["mixer"], d64(W), "l0.mix.", EPS)
    for name, val in (("u", 0.0), ("w0", -30.0), ("mu.k", 0.0)):
        V = dict(d64(W))
        V["l0.mix." + name] = torch.full_like(V["l0.mix." + name], val)
        assert rel_err(O.wkv_mixer(h, l["mixer"], V, "l0.mix.", EPS), want) > 0.05, name
    assert rel_err(run_mixer(l, W, h.float(), target, [(0, 9), (9, 10), (10, 40)]), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(heads=5, kv_heads=5, dim=16, vdim=3), dict(heads=1, kv_heads=1, dim=6),
                                   dict(heads=36, kv_heads=2, diff=0.8), dict(heads=3, kv_heads=1, dim=80, vdim=130),
                                   dict(heads=2, kv_heads=1, dim=40, vdim=24, scale=0.05)])
def test_differential_attention_alone(target, shape):
    l = O.attn_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=5)
    h = rows(90, 24, 3).double()
    want, _ = O.diff_attention_mixer(h, l["mixer"], d64(W), "l0.mix.", EPS)
    for cuts in CUTS:
        assert rel_err(run_mixer(l, W, h.float(), target, cuts), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(heads=4, kv_heads=2, dim=64, vdim=128), dict(heads=2, kv_heads=1, dim=128, vdim=96),
                                   dict(heads=8, kv_heads=1, dim=32, vdim=64), dict(heads=2, kv_heads=2, dim=16, vdim=256)])
def test_differential_attention_head_sizes_of_real_models(target, shape):
    """Head sizes that are multiples of 8 (in bf16 every instantiation of the matrix-core kernel, and the generic
    kernel for the 256-wide values), with enough keys that rows decoded alone split their keys into several runs."""
    l = O.attn_layer(**shape)
    W = O.make_weights(O.make_config([l], width=24), seed=20)
    h = rows(300, 24, 8).double()
    want, _ = O.diff_attention_mixer(h, l["mixer"], d64(W), "l0.mix.", EPS)
    cuts = [(0, 150), (150, 297), (297, 298), (298, 299), (299, 300)]
    (mix,), dev, dt = build_mixers([l], W, target, 24)
    meta0, _ = one_seq_meta(1, dev, total=304)
    cache = torch.zeros(304 // 4 + 3, 4, mix.cache_dim, device=dev, dtype=dt)
    got = []
    for a, b in cuts:
        meta, _ = one_seq_meta(b - a, dev, start=a, total=304)
        meta.max_ctx = b
        got.append(mix.forward(h[a:b].to(dev, dt), meta, cache, None))
    assert rel_err(torch.cat(got), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
def test_second_map_norms_and_biases_matter(target):
    l = O.attn_layer()
    W = O.make_weights(O.make_config([l], width=24), seed=6)
    h = rows(50, 24, 4).double()
    m = l["mixer"]
    want, _ = O.diff_attention_mixer(h, m, d64(W), "l0.mix.", EPS)
    V = d64(W)
    assert abs(O.lam_of(m, V, "l0.mix.") - m["diff"]) > 0.02          # the learned vectors move lam
    for name in ("q.norm", "k.norm", "q.b", "v.b", "o.b", "lq1"):
        U = dict(V)
        U["l0.mix." + name] = torch.ones_like(U["l0.mix." + name]) * (0.0 if name.endswith(".b") else 1.0)
        assert rel_err(O.diff_attention_mixer(h, m, U, "l0.mix.", EPS)[0], want) > 0.01, name
    swapped = dict(V)   # the two maps are not interchangeable
    q = V["l0.mix.q"].view(m["heads"], 2, m["dim"], -1)
    swapped["l0.mix.q"] = q.flip(1).reshape(V["l0.mix.q"].shape)
    assert rel_err(O.diff_attention_mixer(h, m, swapped, "l0.mix.", EPS)[0], want) > 0.05
    assert rel_err(run_mixer(l, W, h.float(), target, [(0, 50)]), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
def test_reader_of_another_layers_keys_and_values_alone(target):
    """Layer 1 has no key / value tensors and reads the cache layer 0 wrote, in portions and token by token."""
    layers = [O.attn_layer(heads=2, kv_heads=2, dim=8, vdim=6), O.attn_layer(heads=6, kv_heads=2, dim=8, vdim=6, diff=0.7, kv_from=0)]
    W = O.make_weights(O.make_config(layers, width=24), seed=7)
    assert "l1.mix.k" not in W and "l1.mix.v.b" not in W and "l1.mix.k.norm" not in W
    h0, h1 = rows(60, 24, 5).double(), rows(60, 24, 6).double()
    _, kv = O.diff_attention_mixer(h0, layers[0]["mixer"], d64(W), "l0.mix.", EPS)
    want, _ = O.diff_attention_mixer(h1, layers[1]["mixer"], d64(W), "l1.mix.", EPS, kv)
    (src, reader), dev, dt = build_mixers(layers, W, target, 24)
    assert reader.cache_dim == 0 and src.cache_dim == 2 * (2 * 8) + 2 * 6
    _, nblk = one_seq_meta(1, dev)
    cache = torch.zeros(nblk, 4, src.cache_dim, device=dev, dtype=dt)
    got = []
    for a, b in [(0, 21), (21, 23), (23, 24), (24, 59), (59, 60)]:
        meta, _ = one_seq_meta(b - a, dev, start=a)
        src.forward(h0[a:b].to(dev, dt), meta, cache, None)
        got.append(reader.forward(h1[a:b].to(dev, dt), meta, cache, None))
    assert rel_err(torch.cat(got), want) < TOL[target[1]]


@pytest.mark.parametrize("target", TARGETS)
def test_state_is_carried_not_reset_and_slots_are_separate(target):
    """Two sequences take turns in two slots; a lost or mixed-up state (or previous row) would show."""
    l = O.wkv_layer()
    W = O.make_weights(O.make_config([l], width=24), seed=8)
    (mix,), dev, dt = build_mixers([l], W, target, 24)
    hs = [rows(30, 24, 10), rows(30, 24, 11)]
    wants = [O.wkv_mixer(h.double(), l["mixer"], d64(W), "l0.mix.", EPS) for h in hs]
    state = [torch.zeros(s, device=dev, dtype=torch.float32) for s in mix.state_shapes(3)]
    got = [[], []]
    for a, b in ((0, 7), (7, 8), (8, 21), (21, 30)):
        for k in (0, 1):
            meta, _ = one_seq_meta(b - a, dev, start=a, slot=2 - k)
            got[k].append(mix.forward(hs[k][a:b].to(dev), meta, None, state))
    for k in (0, 1):
        assert rel_err(torch.cat(got[k]), wants[k]) < TOL[target[1]]
    assert rel_err(torch.cat(got[0]), wants[1]) > 0.3


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("shape", [dict(), dict(experts=1, top=1, identity=0, shared=0), dict(experts=2, top=4, identity=3, scale=0.5),
                                   dict(experts=9, top=2, identity=0, ff=7, shared=33), dict(experts=70, top=5, identity=70, ff=8)])
def test_routed_experts_alone(target, shape):
    """Router (softmax over all outputs, corrected choice, uncorrected weights), gated experts, identity
    experts, shared expert, and the residual update that combines them."""
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    ops = get_ops(dev)
    f = O.moe(**shape)
    cfg = O.make_config([O.wkv_layer(mlp=f)], width=24)
    W = O.make_weights(cfg, seed=9)
    n = f["router"]["experts"] + f["router"]["identity"]
    W["l0.mlp.correction"] = (torch.randn(n, generator=torch.Generator().manual_seed(1)) * 0.3).bfloat16().float()
    h = rows(70, 24, 7)
    V = d64(W)
    y = O.moe_ff(h.double(), f, V, "l0.mlp.")
    # the correction changes which experts are chosen, and the weights are the uncorrected scores
    idx, wgt = O.route(h.double(), f, V, "l0.mlp.")
    if n > f["router"]["top"]:
        U = dict(V)
        U["l0.mlp.correction"] = torch.zeros(n, dtype=torch.float64)
        assert (O.route(h.double(), f, U, "l0.mlp.")[0] != idx).any()
    res0 = rows(70, 24, 8)
    want = res0.double() + O.out_norm(y, V["l0.norm2"], EPS)
    spec = KemavikConfig.from_dict(cfg).layers[0].mlp
    assert isinstance(spec, RoutedMoESpec)
    ff = make_ff(spec, 24, dev, dt, ops)
    ff.load(lambda k: W[k], "l0.mlp.")
    res = res0.to(dev).clone()
    out = torch.empty(70, 24, device=dev, dtype=dt)
    ops.add_normed(out, res, None, (1.0 + W["l0.norm2"]).to(dev), EPS, ff.forward(h.to(dev, dt)))
    tol = 2e-4 if target[1] == "float32" else 3e-2
    assert rel_err(res, want) < tol and rel_err(out, want) < tol
    if target[1] == "float32":   # same choices as the oracle, identity experts in their bucket
        got_ids = ff.forward(h.to(dev, dt))[2].cpu().long()
        assert torch.equal(got_ids.sort(-1).values, idx.clamp(max=f["router"]["experts"]).sort(-1).values)


@pytest.mark.gpu
def test_routed_experts_large_batch_gpu():
    """Enough pairs per expert that the experts run as the packed grouped GEMM of the dense families' prefill
    (gate in its epilogue, the identity bucket's tiles left out)."""
    dev, ops = torch.device("cuda"), get_ops("cuda")
    f = O.moe(experts=2, top=2, ff=256, identity=1, shared=0)
    cfg = O.make_config([O.wkv_layer(mlp=f)], width=256)
    W = O.make_weights(cfg, seed=19)
    h = rows(500, 256, 3)
    y = O.moe_ff(h.double(), f, d64(W), "l0.mlp.")
    ff = make_ff(KemavikConfig.from_dict(cfg).layers[0].mlp, 256, dev, torch.bfloat16, ops)
    ff.load(lambda k: W[k], "l0.mlp.")
    assert ff._packed_ok(h.to(dev, torch.bfloat16), 1000, 3)
    res = torch.zeros(500, 256, device=dev)
    out = torch.empty(500, 256, device=dev, dtype=torch.bfloat16)
    ops.add_normed(out, res, None, torch.ones(256, device=dev), EPS, ff.forward(h.to(dev, torch.bfloat16)))
    assert ff.packed is not None and rel_err(res, O.rms(y, EPS)) < 3e-2


@pytest.mark.parametrize("target", TARGETS)
def test_dense_feed_forward_and_output_norm_alone(target):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    ops = get_ops(dev)
    cfg = O.make_config([O.wkv_layer(mlp=O.dense(ff=50))], width=24)
    W = O.make_weights(cfg, seed=10)
    h = (rows(40, 24, 4) * 2).double()
    want = O.dense_ff(h, d64(W), "l0.mlp.")
    ff = make_ff(KemavikConfig.from_dict(cfg).layers[0].mlp, 24, dev, dt, ops)
    ff.load(lambda k: W[k], "l0.mlp.")
    assert rel_err(ff.forward(h.to(dev, dt)), want) < TOL[target[1]]
    z = torch.linspace(-5, 5, 64).view(1, -1)
    got = torch.empty_like(z, device=dev)
    ops.activation(got, z.to(dev), "relu2")
    assert torch.allclose(got.cpu(), torch.relu(z) ** 2, atol=1e-6)
    gu = rows(3, 32, 9)
    got = torch.empty(3, 16, device=dev)
    ops.activation(got, gu.to(dev), "silu_mul")
    assert torch.allclose(got.cpu(), O.silu(gu[:, :16]) * gu[:, 16:], atol=1e-5)
    # x <- x + norm(y) with a weight stored around zero; the stream stays 32-bit and the copy is rounded once
    res = rows(40, 24, 5).to(dev)
    y = (rows(40, 24, 6) * 5).to(dt)
    w = 0.1 * rows(1, 24, 7)[0]
    x2 = res.cpu().double() + O.out_norm(y.double(), w.double(), EPS)
    out = torch.empty(40, 24, device=dev, dtype=dt)
    ops.add_normed(out, res, y.to(dev), (1.0 + w).to(dev), EPS)
    assert torch.allclose(res.cpu().double(), x2, atol=2e-6)
    assert torch.equal(out.cpu(), res.cpu().to(dt))


@pytest.mark.parametrize("target", TARGETS)
def test_token_shift_alone(target):
    dev, dt = torch.device(target[0]), getattr(torch, target[1])
    ops = get_ops(dev)
    x = rows(12, 300, 1)
    mu = torch.rand(3, 300, generator=torch.Generator().manual_seed(2))
    state = torch.full((3, 300), 5.0, device=dev)
    before = torch.cat([torch.zeros(1, 300), x[:-1]])
    want = x[None] + (before - x)[None] * mu[:, None]
    got = []
    for a, b in ((0, 5), (5, 6), (6, 12)):
        meta, _ = one_seq_meta(b - a, dev, start=a, slot=2)
        out = torch.empty(3, b - a, 300, device=dev, dtype=dt)
        ops.token_shift(out, x[a:b].to(dev), state, mu.to(dev), meta)
        got.append(out.float().cpu())
    assert torch.allclose(torch.cat(got, 1), want.to(dt).float(), atol=1e-6 if target[1] == "float32" else 2e-2)
    assert torch.equal(state[2].cpu(), x[11]) and float(state[1].min()) == 5.0


# ---------------------------------------------------------------- engine
@pytest.mark.parametrize("target", TARGETS)
def test_prefill_and_long_decoding(tmp_path, target):
    cfg = base_config()
    W = O.make_weights(cfg, seed=11)
    toks = tokens(70, cfg["vocab"], 1)
    streams = []
    ref = O.forward(cfg, W, toks, streams)
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
    W = O.make_weights(cfg, seed=12)
    toks = tokens(83, cfg["vocab"], 2)
    ref = O.forward(cfg, W, toks)
    check_all(replay(session(tmp_path, cfg, W, target), portions(toks, sizes)), "a", ref, TOL[target[1]])


@pytest.mark.parametrize("target", TARGETS)
def test_unequal_requests_in_one_batch_and_reuse(tmp_path, target):
    """Up to four live requests of unequal length, portions beside single tokens; finished requests
    give pages and slots back and later ones take them; the pool is small enough that they must."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=13)
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


def planted(far, probes, n, seed, kv_reader):
    """A model whose first layer is attention with keys made from its first head's query weights with the
    columns reversed, so a query scores highest (both maps) against the key of the token whose embedding is
    its own reversed: the probe tokens are paired so with the tokens at the far positions."""
    lay = [O.attn_layer(heads=2, kv_heads=1, dim=32, vdim=8, scale=1.0, mlp=O.dense(24))]
    if kv_reader:
        lay.append(O.attn_layer(heads=2, kv_heads=1, dim=32, vdim=8, scale=1.0, kv_from=0))
    cfg = O.make_config(lay, width=32, vocab=100 + 2 * len(far))
    W = O.make_weights(cfg, seed=seed)
    W["l0.mix.k"] = W["l0.mix.q"][:64].flip(1).clone()
    for s in ("q.b", "k.b"):
        W["l0.mix." + s] = torch.zeros_like(W["l0.mix." + s])
    W["l0.mix.k.norm"] = W["l0.mix.q.norm"].clone()
    toks = [t % 100 for t in tokens(n, 1000, seed)]
    for i, (a, b) in enumerate(zip(far, probes)):
        W["embed"][101 + 2 * i] = W["embed"][100 + 2 * i].flip(0)
        toks[a], toks[b] = 100 + 2 * i, 101 + 2 * i   # token ids used nowhere else
    return cfg, W, toks


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("kv_reader", [False, True])
def test_far_keys_at_page_borders(tmp_path, target, kv_reader):
    """Keys hundreds of tokens back, in the last and the first slot of a page (the replay engine's pages hold
    16 tokens) and at the very first position, asked for from inside a prompt and by tokens decoded alone.
    Changing the far token moves the probe's logits, so a lost or misplaced key shows."""
    far, probes = [0, 47, 48, 175], [300, 317, 322, 325]
    cfg, W, toks = planted(far, probes, 330, 15, kv_reader)
    ref = O.forward(cfg, W, toks)
    for a, b in zip(far, probes):
        other = list(toks)
        other[a] = 7
        assert rel_err(O.forward(cfg, W, other)[b:b + 1], ref[b:b + 1]) > 0.1
    sess = session(tmp_path, cfg, W, target)
    tol = TOL[target[1]] * (1 if target[1] == "float32" else 2)   # scores near 30: bf16 rounds them by 0.1 and more
    check_all(replay(sess, portions(toks, [330])), "a", ref, tol)
    check_all(replay(sess, portions(toks, [129, 64, 107, 2, 18, 2])), "a", ref, tol)   # 300, 322, 325 in portions; 317 alone
    check_all(replay(sess, portions(toks, [299])), "a", ref, tol)                      # every probe decoded alone


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("variant", ["ones", "no_mlp", "readers", "wide", "unequal", "odd"])
def test_other_sizes(tmp_path, target, variant):
    d = O.dense(ff=8)
    if variant == "ones":           # everything 1 that can be
        layers = [O.attn_layer(heads=1, kv_heads=1, dim=8, vdim=8, mlp=O.moe(experts=1, top=1, identity=1, shared=0)),
                  O.wkv_layer(heads=1, dim=8, mlp=d), O.attn_layer(heads=1, kv_heads=1, dim=8, vdim=8, kv_from=0)]
        cfg = O.make_config(layers, width=16, vocab=50)
    elif variant == "no_mlp":
        layers = [O.wkv_layer(), O.attn_layer(heads=7, kv_heads=7, dim=4, vdim=20), O.wkv_layer(heads=4, dim=3)]
        cfg = O.make_config(layers, width=48)
    elif variant == "readers":      # several readers of one layer, one of them past a linear-attention layer; a second source
        layers = [O.attn_layer(mlp=d), O.attn_layer(kv_from=0, diff=0.2, mlp=O.moe(top=4, identity=4)),
                  O.wkv_layer(mlp=d), O.attn_layer(heads=2, kv_from=0, diff=0.9), O.attn_layer(vdim=4, scale=0.9, mlp=d),
                  O.attn_layer(heads=8, vdim=4, kv_from=4, mlp=d)]
        cfg = O.make_config(layers, width=36)
    elif variant == "wide":         # head sizes that are no multiples of 8, 16 or 64, value heads wider than key heads
        layers = [O.attn_layer(heads=2, kv_heads=1, dim=72, vdim=136, mlp=O.dense(ff=70)), O.wkv_layer(heads=2, dim=66),
                  O.attn_layer(heads=2, kv_heads=2, dim=20, vdim=7, mlp=O.moe(experts=3, ff=65, shared=9))]
        cfg = O.make_config(layers, width=24)
    elif variant == "odd":          # nothing a multiple of 4; experts on a linear-attention layer
        layers = [O.wkv_layer(heads=3, dim=5, mlp=O.moe(experts=3, top=2, identity=1, ff=7, shared=5)),
                  O.attn_layer(heads=3, kv_heads=1, dim=6, vdim=5, mlp=O.dense(ff=11)), O.attn_layer(heads=9, kv_heads=1, dim=6, vdim=5, kv_from=1)]
        cfg = O.make_config(layers, width=30, vocab=53)
    else:                           # heads * vdim, 2 * heads * dim and the width all differ; vdim < dim; group of 3
        layers = [O.attn_layer(heads=6, kv_heads=2, dim=16, vdim=8, mlp=O.moe(experts=6, top=2, identity=0, ff=20, shared=12)),
                  O.wkv_layer(heads=3, dim=16, mlp=O.dense(ff=100))]
        cfg = O.make_config(layers, width=40, vocab=77, eps=1e-3)
    W = O.make_weights(cfg, seed=17)
    toks = tokens(45, cfg["vocab"], 5)
    ref = O.forward(cfg, W, toks)
    sess = session(tmp_path, cfg, W, target)
    check_all(replay(sess, portions(toks, [45])), "a", ref, TOL[target[1]])
    check_all(replay(sess, portions(toks, [4, 9, 2, 13])), "a", ref, TOL[target[1]])


def test_config_reader():
    cfg = base_config(eps=3e-4)
    c = KemavikConfig.from_dict(cfg)
    assert c.norm_eps == 3e-4 and c.num_layers == 6 and [r[0] for r in c.runs()] == list(range(6))
    w, a, r = c.layers[0].mixer, c.layers[1].mixer, c.layers[2].mixer
    assert isinstance(w, WkvSpec) and (w.heads, w.dim) == (3, 8)
    assert isinstance(a, WindowAttentionSpec) and (a.maps, a.head_norm, a.bias, a.out_bias, a.sink, a.gate) == (2, True, True, True, False, False)
    assert (a.diff, a.window, a.rot_dims, a.kv_from, a.cache_dim) == (0.3, 0, 0, None, 2 * 2 * 8 + 2 * 12)
    assert r.kv_from == 1 and r.cache_dim == 0
    f = c.layers[1].mlp
    assert (f.experts, f.top, f.ff, f.identity, f.scale, f.shared_ff) == (5, 2, 12, 2, 1.5, 20)
    assert c.layers[4].mlp is None and c.layers[0].mlp.act == "relu2"
    for j in (2, 0, 5):   # itself, a layer that is no attention, a later layer
        bad = base_config()
        bad["layers"][2] = O.attn_layer(kv_from=j)
        with pytest.raises(ValueError):
            KemavikConfig.from_dict(bad)
    bad = base_config()
    bad["layers"][2] = O.attn_layer(kv_heads=1, kv_from=1)   # other key / value heads than its source
    with pytest.raises(ValueError):
        KemavikConfig.from_dict(bad)


@pytest.mark.parametrize("target", TARGETS)
def test_greedy_generation_through_the_scheduler(tmp_path, target):
    """LLMEngine.generate: the scheduler's own chunked prefill (a 24-token budget), batching of three
    prompts of unequal length and the sampler; every generated token is an argmax of the oracle's
    logits over the tokens before it."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=18)
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
        lg = O.forward(cfg, W, p + out)
        for k, t in enumerate(out):
            row = lg[len(p) + k - 1]
            assert row[t] >= row.max() - slack, (k, t, int(row.argmax()))
    assert eng.states.num_free() == 4 and eng.blocks.num_free() == eng.blocks.num_blocks


@pytest.mark.gpu
def test_graph_decode_matches_eager_gpu(tmp_path):
    """Decode-only steps replay a captured hipGraph (state slots and block tables staged per step): same
    greedy tokens as the eager engine, and argmaxes of the oracle."""
    cfg = base_config()
    W = O.make_weights(cfg, seed=23)
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
        lg = O.forward(cfg, W, p + out)
        for k, t in enumerate(out):
            row = lg[len(p) + k - 1]
            assert row[t] >= row.max() - 0.3, (k, t, int(row.argmax()))   # logits of +-7 after 20 bf16 steps
    same = sum(a == b for a, b in zip(outs[0], outs[1]))
    assert same >= len(prompts) - 1, (outs[0], outs[1])  # bf16 near-ties may flip one continuation


def test_preset_and_cli_model_resolution(tmp_path):
    from hipserve.config import resolve_model_config
    from hipserve.models.registry import model_class

    cfg = base_config()
    path = O.save_checkpoint(str(tmp_path / "c"), cfg, O.make_weights(cfg, seed=1))
    m = resolve_model_config(path)
    assert isinstance(m, KemavikConfig) and model_class(m).__name__ == "KemavikModel"
    t = resolve_model_config("tiny-kemavik")
    assert isinstance(t, KemavikConfig) and t.layers[2].mixer.kv_from == 1
