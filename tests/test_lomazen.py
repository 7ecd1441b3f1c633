"""Lomazen model family: the framework's ragged engine path against a plain
per-sequence oracle (tests/lomazen_oracle.py) on small random configurations.

Covers each mechanism alone (norms on both sides of a sublayer, the restart of
the repeated block, rotation frequencies and both pairings, gated capped
attention, differential attention, both feed-forwards, the router), prefill
against token-by-token decoding, prompt portions down to two tokens, mixed
batches against each request alone, reuse of freed pages and slots, keys far
away and at page borders in prompts and in decoding (planted so that a lost key
shows), a cap that matters, the first tokens of a sequence, long decoding,
degenerate and unequal sizes, and greedy generation through the engine's own
scheduler.
"""

import copy
import json
import math
import os

import pytest
import torch

import lomazen_oracle as O
from megatron_amd.inference import DynamicInferenceEngine, SamplingParams
from megatron_amd.inference.contexts import HybridInferenceContext
from megatron_amd.models.lomazen import LomazenConfig, LomazenModel, load_lomazen_state

F64 = torch.float64
SCALING = dict(factor=3.0, low=2.0, high=5.0, original=40)


def att(heads=4, kv=2, dim=6, vdim=5, rot=4, base=100.0, scale=0.6, cap=4.0, scaling=SCALING, mlp="moe", experts=5,
        top=2, ff=9):
    m = dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale)
    if cap:
        m["softcap"] = cap
    if rot:
        m["rot"] = dict(dims=rot, base=base)
        if scaling:
            m["rot"]["scaling"] = dict(scaling)
    return dict(type="attention", mixer=m, mlp=_mlp(mlp, experts, top, ff))


def att2(heads=2, kv=1, dim=4, vdim=7, rot=2, base=30.0, scale=0.7, diff=0.3, mlp="dense", experts=4, top=3, ff=11):
    m = dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale, diff=diff)
    if rot:
        m["rot"] = dict(dims=rot, base=base)
    return dict(type="attention_2", mixer=m, mlp=_mlp(mlp, experts, top, ff))


def _mlp(kind, experts, top, ff):
    if kind is None:
        return None
    if kind == "dense":
        return dict(kind="dense", ff=ff)
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


def make_config(layers, width=24, vocab=41, eps=1e-5, loop=(1, 3, 2), logit_scale=1.5):
    cfg = dict(architecture="Lomazen", vocab=vocab, width=width, norm=dict(eps=eps), layers=copy.deepcopy(layers))
    if loop:
        cfg["loop"] = dict(start=loop[0], stop=loop[1], times=loop[2])
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    return cfg


def make_weights(cfg, seed=0, gain=1.0):
    """Random checkpoint tensors under the checkpoint's names (bf16-representable
    values so that both sides read the same numbers)."""
    g = torch.Generator().manual_seed(seed)
    W, out = cfg["width"], {}

    def rnd(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16).float()

    def lin(o, i):
        return rnd(o, i, scale=gain / math.sqrt(i))

    out["embed"] = rnd(cfg["vocab"], W)
    if cfg.get("loop"):
        out["loop.in"] = lin(W, 2 * W) * 1.5
        out["loop.step"] = rnd(cfg["loop"]["times"], W, scale=0.5)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        a = p + "mix."
        out[p + "norm1"], out[p + "norm1b"] = 1 + rnd(W, scale=0.2), 1 + rnd(W, scale=0.2)
        H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
        if L["type"] == "attention":
            out[a + "q"], out[a + "k"], out[a + "v"] = lin(H * d, W) * 2, lin(G * d, W) * 2, lin(G * e, W)
            out[a + "g"], out[a + "o"] = lin(H * e, W) * 2, lin(W, H * e)
        else:
            out[a + "q"], out[a + "k"], out[a + "v"] = lin(H * 2 * d, W) * 2, lin(G * 2 * d, W) * 2, lin(G * e, W)
            out[a + "g"], out[a + "o"] = lin(H, W) * 2, lin(W, H * e)
            for nm in ("lq1", "lk1", "lq2", "lk2"):
                out[a + nm] = rnd(d, scale=0.4)
        if L.get("mlp"):
            mm, q = L["mlp"], p + "mlp."
            out[p + "norm2"], out[p + "norm2b"] = 1 + rnd(W, scale=0.2), 1 + rnd(W, scale=0.2)
            if mm["kind"] == "dense":
                out[q + "gate"], out[q + "up"], out[q + "down"] = lin(mm["ff"], W) * 2, lin(mm["ff"], W) * 2, lin(W, mm["ff"])
            else:
                E, ff = mm["router"]["experts"], mm["expert"]["ff"]
                out[q + "router"] = lin(E, W) * 3
                for e_ in range(E):
                    out[f"{q}e{e_}.up"], out[f"{q}e{e_}.down"] = lin(ff, W) * 2, lin(W, ff)
    out["final.norm"] = 1 + rnd(W, scale=0.2)
    return {k: v.to(torch.bfloat16).float() for k, v in out.items()}


def build(cfg, weights, dtype=torch.float32, device="cpu"):
    model = LomazenModel(LomazenConfig.from_dict(cfg, dtype=dtype))
    load_lomazen_state(model, weights)
    return model.to(device).eval()


def oracle(cfg, w, toks, trace=None):
    return O.model(toks, cfg, w, trace)


def engine_for(model, pages=40, page=8, slots=4, **kw):
    return DynamicInferenceEngine(model, num_blocks=pages, block_size=page, max_batch=slots,
                                  use_hip_graphs=False, enable_prefix_caching=False, **kw)


def tokens_of(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def feed(engine, req, toks):
    """All positions' logits of one feed."""
    return engine.forward_batch([(req, toks)], [list(range(len(toks)))])


def assert_close(got, want, tol=2e-4):
    want = want.float()
    scale = want.abs().max().item()
    err = (got.detach().cpu().float() - want).abs().max().item()
    assert err <= tol * max(scale, 1.0), f"max abs error {err} (scale {scale})"


def run_in_portions(engine, toks, cuts):
    """Feed toks in portions of the given sizes (the rest one by one); all logits."""
    req = engine.open_request()
    out, at = [], 0
    for c in cuts:
        c = min(c, len(toks) - at)
        if c <= 0:
            break
        out.append(feed(engine, req, toks[at:at + c]))
        at += c
    while at < len(toks):
        out.append(feed(engine, req, toks[at:at + 1]))
        at += 1
    engine.close_request(req)
    return torch.cat(out, dim=0)


# one layer ahead of the repeated block, two inside it (both kinds), two behind it, one without a feed-forward
FULL = [att(mlp="dense"), att2(mlp="moe"), att(heads=6, kv=2, dim=4, vdim=3, rot=2, cap=None, scaling=None),
        att2(heads=4, kv=4, dim=6, vdim=2, rot=6, diff=0.55, mlp=None), att(kv=1, rot=0, top=5)]


# -- each mechanism alone ------------------------------------------------------


def test_norms_around_a_sublayer_and_restart():
    from megatron_amd.ops import ragged as R

    torch.manual_seed(0)
    T, W = 7, 24
    x = torch.randn(T, W) * 2
    cur = x.double()
    for k in range(3):
        y, wp, wn = torch.randn(T, W) * 3, 1 + torch.randn(W) * 0.2, 1 + torch.randn(W) * 0.2
        h = R.sandwich_norm_add(x, y, wp, wn, 1e-5, torch.float32)
        cur = cur + O.rms_norm(y.double(), wp.double(), 1e-5)
        assert_close(x, cur, 1e-6)
        assert_close(h, O.rms_norm(cur, wn.double(), 1e-5), 1e-6)
    wide = torch.zeros(T, 2 * W)
    assert R.sandwich_norm_add(x, None, None, None, 1e-5, torch.float32, copy_to=wide[:, :W]) is None
    assert torch.equal(wide[:, :W], x) and not wide[:, W:].any()
    y, b, wn = torch.randn(T, W), torch.randn(W), 1 + torch.randn(W) * 0.2
    x2, h2 = R.restart_norm(y, b, wn, 1e-5, torch.float32)
    assert_close(x2, y.double() + b.double(), 1e-6)
    assert_close(h2, O.rms_norm(y.double() + b.double(), wn.double(), 1e-5), 1e-6)


def test_rotation_frequencies_take_all_three_branches():
    from megatron_amd.ops import ragged as R

    rot = dict(dims=16, base=1000.0, scaling=dict(factor=8.0, low=1.0, high=3.0, original=64))
    want = O.rotation_freqs(rot)
    plain = O.rotation_freqs(dict(dims=16, base=1000.0))
    kinds = {"kept" if a == b else ("divided" if abs(a - b / 8.0) < 1e-15 else "blended") for a, b in zip(want, plain)}
    assert kinds == {"kept", "divided", "blended"}
    got = R.scaled_freqs(16, 1000.0, rot["scaling"])
    assert_close(got, torch.tensor(want, dtype=F64), 1e-7)
    assert_close(R.scaled_freqs(16, 1000.0, None), torch.tensor(plain, dtype=F64), 1e-7)
    assert R.scaled_freqs(0, 10.0, None).numel() == 0


@pytest.mark.parametrize("layout", ["pairs", "halves"])
@pytest.mark.parametrize("D,rot", [(8, 8), (8, 4), (7, 2), (6, 0)])
def test_rotation_pairings(layout, D, rot):
    from megatron_amd.ops import ragged_reference as ref

    torch.manual_seed(1)
    n = 19
    x = torch.randn(n, 3, D)
    fr = O.rotation_freqs(dict(dims=rot, base=50.0)) if rot else []
    want = O.rotate(x.double(), fr, layout)
    got = ref._rotate_layout(x, torch.arange(n), torch.tensor(fr, dtype=torch.float32), layout)
    assert_close(got, want, 1e-5)
    if rot:
        other = O.rotate(x.double(), fr, "halves" if layout == "pairs" else "pairs")
        assert (rot == 2) == bool((want - other).abs().max() < 1e-9)      # with one pair the two pairings agree


def _module_ctx(caches, n, page, dtype=torch.float32, device="cpu"):
    pages = (n + page - 1) // page
    ctx = HybridInferenceContext(caches, {}, pages + 2, page, 2, dtype=dtype, device=device)
    ctx.allocator.allocate(1)
    table = ctx.allocator.allocate(pages)[::-1]
    return ctx, table, ctx.acquire_slot()


def _r(g, *s):
    return torch.randn(*s, generator=g)


@pytest.mark.parametrize("H,G,D,V,rot,cap,scaling", [(4, 2, 6, 5, 4, 4.0, SCALING), (3, 3, 4, 4, 4, None, None),
                                                     (2, 1, 8, 3, 0, 2.0, None), (4, 4, 4, 6, 2, 40.0, SCALING),
                                                     (6, 2, 2, 2, 2, 1.0, None), (1, 1, 10, 1, 6, None, SCALING),
                                                     (4, 1, 5, 4, 4, 3.0, None)])
def test_gated_attention_alone(H, G, D, V, rot, cap, scaling):
    from megatron_amd.transformer.gated_softcap_attention import GatedSoftcapAttention

    g = torch.Generator().manual_seed(3)
    W, n, page = 16, 45, 8
    m = att(H, G, D, V, rot, 50.0, 1.5, cap, scaling)["mixer"]
    wt = {"q": _r(g, H * D, W) / 2, "k": _r(g, G * D, W) / 2, "v": _r(g, G * V, W) / 4, "g": _r(g, H * V, W) / 2,
          "o": _r(g, W, H * V) / 4}
    mod = GatedSoftcapAttention(W, H, G, D, V, 1.5, 1e-5, softcap=cap, rot_dims=rot, rot_base=50.0, rot_scaling=scaling,
                                layout="pairs", unit_norm=True, dtype=torch.float32)
    with torch.no_grad():
        mod.w_in.copy_(torch.cat([wt["q"], wt["k"], wt["v"], wt["g"]]))
        mod.w_out.copy_(wt["o"])
    h = _r(g, n, W)
    want = O.gated_attention(h.double(), {k: v.double() for k, v in wt.items()}, m, 1e-5)
    ctx, table, slot = _module_ctx(mod.cache_spec("a", page), n, page)
    got, at = [], 0
    for c in (19, 2, 1, 13, 10):
        ctx.begin_batch([c], [at], [slot], [table])
        with torch.no_grad():
            got.append(mod(h[at:at + c], ctx, "a"))
        at += c
    assert at == n
    assert_close(torch.cat(got), want, 1e-5)


@pytest.mark.parametrize("H,G,D,V,rot,diff", [(2, 1, 4, 7, 2, 0.3), (3, 3, 6, 4, 6, 0.8), (4, 2, 8, 3, 0, 0.1),
                                              (1, 1, 2, 1, 2, 0.5), (6, 2, 4, 5, 4, 0.65)])
def test_differential_attention_alone(H, G, D, V, rot, diff):
    from megatron_amd.transformer.differential_attention import DifferentialAttention

    g = torch.Generator().manual_seed(4)
    W, n, page = 16, 41, 8
    m = att2(H, G, D, V, rot, 20.0, 0.9, diff)["mixer"]
    wt = {"q": _r(g, H * 2 * D, W) / 2, "k": _r(g, G * 2 * D, W) / 2, "v": _r(g, G * V, W) / 4, "g": _r(g, H, W) / 2,
          "o": _r(g, W, H * V) / 4, "lq1": _r(g, D) / 2, "lk1": _r(g, D) / 2, "lq2": _r(g, D) / 2, "lk2": _r(g, D) / 2}
    mod = DifferentialAttention(W, H, G, D, V, 0.9, 1e-5, diff, rot_dims=rot, rot_base=20.0, layout="halves",
                                dtype=torch.float32)
    with torch.no_grad():
        mod.w_in.copy_(torch.cat([wt["q"], wt["k"], wt["v"], wt["g"]]))
        mod.w_out.copy_(wt["o"])
        for nm in ("lq1", "lk1", "lq2", "lk2"):
            getattr(mod, nm).copy_(wt[nm])
    h = _r(g, n, W)
    want = O.differential_attention(h.double(), {k: v.double() for k, v in wt.items()}, m, 1e-5)
    lam = math.exp(float(wt["lq1"] @ wt["lk1"])) - math.exp(float(wt["lq2"] @ wt["lk2"])) + diff
    assert abs(mod.lam().item() - lam) < 1e-5
    ctx, table, slot = _module_ctx(mod.cache_spec("a", page), n, page)
    got, at = [], 0
    for c in (17, 2, 1, 12, 9):
        ctx.begin_batch([c], [at], [slot], [table])
        with torch.no_grad():
            got.append(mod(h[at:at + c], ctx, "a"))
        at += c
    assert_close(torch.cat(got), want, 1e-5)


@pytest.mark.parametrize("E,top", [(6, 2), (8, 1), (5, 5), (9, 3)])
def test_router_alone(E, top):
    """the weights are the chosen experts' scores over ALL experts: they sum to one only when all are chosen"""
    from megatron_amd.ops import ragged as R

    torch.manual_seed(3)
    h, wr = torch.randn(50, 16), torch.randn(E, 16)
    s = torch.softmax(h.double() @ wr.double().T, -1)
    wt, idx = s.topk(top, -1)
    ids, w, _ = R.moe_router(h, wr, E, top, 1, 1, 1.0, None, "softmax_all")
    o1, o2 = idx.argsort(1), ids.long().argsort(1)
    assert torch.equal(idx.gather(1, o1), ids.long().gather(1, o2))
    assert_close(w.gather(1, o2), wt.gather(1, o1), 1e-6)
    assert (abs(w.sum(1) - 1) < 1e-5).all() == (top == E)


@pytest.mark.parametrize("kind", ["dense", "moe"])
def test_feed_forward_alone(kind):
    cfg = make_config([att(mlp=kind)], loop=None)
    w = make_weights(cfg, seed=4)
    layer = build(cfg, w).layers[0]
    torch.manual_seed(5)
    h = torch.randn(21, cfg["width"])
    with torch.no_grad():
        got = layer.mlp(h)
    p = O.sub(w, "l0.mlp.")
    want = O.dense_ff(h.double(), p) if kind == "dense" else O.routed_ff(h.double(), p, cfg["layers"][0]["mlp"])
    assert_close(got, want, 1e-5)


@pytest.mark.parametrize("spec", [att(), att(mlp=None), att(kv=4, mlp="dense"), att(kv=1, cap=None), att(rot=6, top=5),
                                  att(rot=0, top=1), att2(), att2(mlp="moe"), att2(mlp=None, heads=1, kv=1),
                                  att2(heads=4, kv=1, rot=4, diff=0.9)],
                         ids=["att", "att-no-ff", "mha-dense", "mqa-no-cap", "rot-all-top-all", "no-rot-top1", "att2",
                              "att2-moe", "att2-no-ff", "att2-mqa"])
@pytest.mark.parametrize("loop", [None, (0, 1, 1), (0, 1, 3)], ids=["once", "block-of-1-once", "block-of-1-thrice"])
def test_single_layer_matches_oracle(spec, loop):
    cfg = make_config([spec], loop=loop)
    w = make_weights(cfg, seed=1)
    toks = tokens_of(37, cfg["vocab"], 2)
    got = build(cfg, w)(torch.tensor([toks]))[:, 0]
    assert_close(got, oracle(cfg, w, toks))


# -- whole model through the engine -------------------------------------------------


def test_layers_match_oracle():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=6)
    toks = tokens_of(40, cfg["vocab"], 7)
    model = build(cfg, w)
    model.layer_trace = []
    eng = engine_for(model)
    req = eng.open_request()
    got = feed(eng, req, toks)
    trace = []
    want = oracle(cfg, w, toks, trace)
    assert len(model.layer_trace) == len(trace) == len(FULL) + 2        # layers 1, 2 run twice
    for a, b in zip(model.layer_trace, trace):
        assert_close(a, b)
    assert_close(got, want)
    assert set(model.inference_spec(8).caches) == {"l0", "l1.p0", "l1.p1", "l2.p0", "l2.p1", "l3", "l4"}


def test_every_pass_has_its_own_cache_and_step_vector():
    """the same token stream with the step vectors of the passes exchanged, or one pass more, gives other logits"""
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=6)
    toks = tokens_of(12, cfg["vocab"], 7)
    a = oracle(cfg, w, toks)
    w2 = dict(w)
    w2["loop.step"] = w["loop.step"].flip(0)
    b = oracle(cfg, w2, toks)
    assert (a - b).abs().max() > 1e-2
    eng = engine_for(build(cfg, w2))
    assert_close(run_in_portions(eng, toks, [5, 2]), b)


def test_prefill_then_decode_token_by_token():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=8)
    toks = tokens_of(48, cfg["vocab"], 9)
    want = oracle(cfg, w, toks)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, [20]), want)          # 20 at once, then 28 single tokens
    assert_close(run_in_portions(eng, toks, []), want)            # everything token by token


@pytest.mark.parametrize("cuts", [[2, 2, 2, 3, 5, 2, 17, 2], [7, 1, 1, 9, 4, 4, 11], [31, 2], [3] * 16])
def test_portions(cuts):
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=10)
    toks = tokens_of(47, cfg["vocab"], 11)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, cuts), oracle(cfg, w, toks))


def test_mixed_batch_equals_each_alone():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=12)
    model = build(cfg, w)
    seqs = [tokens_of(n, cfg["vocab"], 20 + n) for n in (29, 7, 18, 3)]
    want = [oracle(cfg, w, s) for s in seqs]
    eng = engine_for(model, pages=12)
    reqs = [eng.open_request() for _ in seqs]
    at = [0] * len(seqs)
    got = [[] for _ in seqs]
    plan = [(5, 1, 2, 3), (2, 1, 0, 0), (1, 1, 7, 0), (9, 1, 1, 0), (1, 1, 1, 0), (11, 2, 7, 0)]
    for step in plan:
        feeds, wants, who = [], [], []
        for r, c in enumerate(step):
            c = min(c, len(seqs[r]) - at[r])
            if c > 0:
                feeds.append((reqs[r], seqs[r][at[r]:at[r] + c]))
                wants.append(list(range(c)))
                who.append((r, c))
                at[r] += c
        out = eng.forward_batch(feeds, wants)
        o = 0
        for r, c in who:
            got[r].append(out[o:o + c])
            o += c
    for r in range(len(seqs)):
        assert at[r] == len(seqs[r])
        assert_close(torch.cat(got[r]), want[r])


def test_freed_pages_and_slots_are_reused():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=13)
    eng = engine_for(build(cfg, w), pages=5, page=8, slots=2)     # room for one 40-token request at a time
    for seed in (30, 31, 32):
        toks = tokens_of(33 + seed % 3, cfg["vocab"], seed)
        assert_close(run_in_portions(eng, toks, [9, 2, 12]), oracle(cfg, w, toks))
    a, b = eng.open_request(), eng.open_request()                 # both slots, used before
    ta, tb = tokens_of(11, cfg["vocab"], 40), tokens_of(17, cfg["vocab"], 41)
    out = eng.forward_batch([(a, ta), (b, tb)], [list(range(11)), list(range(17))])
    assert_close(out[:11], oracle(cfg, w, ta))
    assert_close(out[11:], oracle(cfg, w, tb))


# -- edges -----------------------------------------------------------------------------


def test_the_cap_shows():
    """scores far above the cap: leaving the cap out moves the logits well beyond the tolerance"""
    spec = att(heads=2, kv=1, dim=8, vdim=6, rot=4, scale=6.0, cap=1.5, mlp=None)
    cfg = make_config([spec], loop=None)
    w = make_weights(cfg, seed=14)
    toks = tokens_of(30, cfg["vocab"], 15)
    a = oracle(cfg, w, toks)
    other = copy.deepcopy(cfg)
    del other["layers"][0]["mixer"]["softcap"]
    assert (a - oracle(other, w, toks)).abs().max().item() > 50 * 2e-4 * a.abs().max().item()
    for page in (4, 8):
        eng = engine_for(build(cfg, w), pages=16, page=page)
        for cuts in ([], [2] * 15, [30], [4, 1, 5, 6, 4, 10]):
            assert_close(run_in_portions(eng, toks, cuts), a)


def _planted(n, H, G, M, D, V, target, seed):
    """q, k, v of one sequence in which the LAST query's maps all match the key at ``target`` far better than any other"""
    g = torch.Generator().manual_seed(seed)
    q, k, v = _r(g, n, H * M, D), _r(g, n, G * M, D), _r(g, n, G, V)
    rep = H // G
    for qh in range(H * M):
        kh = (qh // (rep * M)) * M + qh % M
        q[n - 1, qh] = 6.0 * k[target, kh] / k[target, kh].norm()
    k[target] *= 3.0
    return q, k, v


@pytest.mark.parametrize("n,target", [(300, 0), (300, 3), (290, 194), (65, 64), (65, 63), (130, 128), (130, 127), (130, 129)])
@pytest.mark.parametrize("maps", [1, 2])
@pytest.mark.parametrize("decode", [False, True])
def test_far_and_border_keys_in_the_attention_op(n, target, maps, decode):
    """a key far back among hundreds, the first key, keys on both sides of a page border and the query's own key;
    the last query is either the end of a prompt portion or a token decoded alone"""
    from megatron_amd.ops import ragged as R

    H, G, D, V, page = 4, 2, 8, 5, 16
    q, k, v = _planted(n, H, G, maps, D, V, target, 5)
    rep = H // G
    want = torch.zeros(n, H * maps, V, dtype=F64)
    for qh in range(H * maps):
        kh, vh = (qh // (rep * maps)) * maps + qh % maps, qh // (rep * maps)
        want[:, qh] = O.causal_softmax(q[:, qh].double() @ k[:, kh].double().T) @ v[:, vh].double()
    ctx, table, slot = _module_ctx({"c": G * (maps * D + V)}, n, page)
    rows = torch.cat([k.reshape(n, -1), v.reshape(n, -1)], dim=1)
    cuts = [n - 1, 1] if decode else [n - 40, 40]
    at, got = 0, []
    for c in cuts:
        batch = ctx.begin_batch([c], [at], [slot], [table])
        ctx.pools["c"][batch.tok_row] = rows[at:at + c]
        got.append(R.map_attention(q[at:at + c].reshape(c, -1), ctx.pools["c"], H, G, maps, D, V, 1.0, 0.0, batch))
        at += c
    got = torch.cat(got)
    assert_close(got, want.reshape(n, -1), 1e-5)
    last = got[-1].view(H * maps, V)                      # the planted key dominates the last row
    own = torch.stack([v[target, qh // (rep * maps)] for qh in range(H * maps)])
    assert (last - own).abs().max().item() < 0.15


def test_rotation_far_from_the_start():
    """one layer whose scores rest on the rotation alone (q = k = a constant vector): position 350 must find
    the keys at the right distance"""
    from megatron_amd.ops import ragged_reference as ref

    n, D = 360, 8
    fr = O.rotation_freqs(dict(dims=D, base=20.0))
    x = torch.ones(n, 1, D)
    for layout in ("pairs", "halves"):
        want = O.rotate(x.double(), fr, layout)
        got = ref._rotate_layout(x, torch.arange(n), torch.tensor(fr, dtype=torch.float32), layout)
        s_want = want[350, 0] @ want[:351, 0].T
        s_got = got[350, 0].double() @ got[:351, 0].double().T
        assert (s_want - s_got).abs().max() < 2e-3 and s_want.argmax() == 350


@pytest.mark.parametrize("n", [1, 2, 3])
def test_first_tokens(n):
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=17)
    toks = tokens_of(n, cfg["vocab"], 18)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, [n]), oracle(cfg, w, toks))
    assert_close(run_in_portions(eng, toks, []), oracle(cfg, w, toks))


def test_long_decoding():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=19)
    toks = tokens_of(100, cfg["vocab"], 20)
    eng = engine_for(build(cfg, w), pages=14)
    assert_close(run_in_portions(eng, toks, [5]), oracle(cfg, w, toks), 3e-4)


@pytest.mark.parametrize("layers,width,vocab,loop,ls", [
    ([att(heads=1, kv=1, dim=2, vdim=1, rot=2, experts=1, top=1, ff=1), att2(heads=1, kv=1, dim=2, vdim=1, rot=2, ff=1)], 8, 5,
     (0, 2, 1), None),
    ([att2(), att2(mlp="moe"), att2(mlp=None)], 16, 30, (2, 3, 3), 0.5),
    ([att(mlp=None), att(heads=3, kv=3, dim=3, vdim=2, rot=2, experts=3, top=3)], 12, 17, None, 1.0),
    ([att(heads=8, kv=4, dim=4, vdim=4, rot=4, experts=2, top=2), att2(heads=4, kv=4, dim=4, vdim=4, rot=4)], 32, 64,
     (0, 2, 2), 2.5),
    ([att(), att2(), att(cap=None)], 20, 33, (1, 2, 4), 1.0),
], ids=["all-ones", "only-differential-late-block", "only-gated-no-block", "equal-sizes-whole-stack-repeats", "block-in-the-middle"])
def test_other_sizes(layers, width, vocab, loop, ls):
    cfg = make_config(layers, width=width, vocab=vocab, loop=loop, logit_scale=ls)
    w = make_weights(cfg, seed=21)
    toks = tokens_of(29, vocab, 22)
    eng = engine_for(build(cfg, w))
    assert_close(run_in_portions(eng, toks, [6, 2, 9]), oracle(cfg, w, toks))


# -- entry points ----------------------------------------------------------------------


def test_greedy_generation_through_the_scheduler():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=23)
    model = build(cfg, w)
    prompts = [tokens_of(n, cfg["vocab"], 50 + n) for n in (13, 4, 21, 9, 2)]   # more requests than slots
    eng = engine_for(model, pages=16, slots=3, max_prefill_tokens=10)            # prompts go in in portions
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, stop_on_eod=False))
    for p, r in zip(prompts, res):
        seq = list(p)
        for tok in r.output_tokens:
            logits = oracle(cfg, w, seq)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() > 1e-3:                                # a near-tie may go either way
                assert tok == int(logits.argmax())
            seq.append(tok)
        assert len(r.output_tokens) == 7


def test_registry_builds_from_a_directory(tmp_path):
    from safetensors.torch import save_file

    from megatron_amd.models.registry import build_from_dir

    cfg = make_config(FULL)
    w = make_weights(cfg, seed=24)
    with open(os.path.join(tmp_path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}, os.path.join(tmp_path, "model.safetensors"))
    model = build_from_dir(str(tmp_path), dtype=torch.float32)
    toks = tokens_of(20, cfg["vocab"], 25)
    assert_close(model(torch.tensor([toks]))[:, 0], oracle(cfg, w, toks))


def test_trace_replay(tmp_path):
    """the replay runner drives the same step function: two requests fed in unequal portions, one ended early"""
    import io

    import numpy as np

    from megatron_amd.inference.trace import replay

    cfg = make_config(FULL)
    w = make_weights(cfg, seed=26)
    eng = engine_for(build(cfg, w))
    a, b = tokens_of(12, cfg["vocab"], 27), tokens_of(9, cfg["vocab"], 28)
    steps = [dict(step=0, entries=[dict(id="a", tokens=a[:7], want=[6]), dict(id="b", tokens=b[:2], want=[])], end=[]),
             dict(step=1, entries=[dict(id="b", tokens=b[2:], want=[0, 6])], end=["b"]),
             dict(step=2, entries=[dict(id="a", tokens=a[7:], want=[4])], end=["a"])]
    log = io.StringIO()
    replay(eng, [json.dumps(s) for s in steps], str(tmp_path), log)
    assert log.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    V = cfg["vocab"]
    r = [torch.from_numpy(np.fromfile(os.path.join(tmp_path, f"{i}.f32"), dtype="<f4").reshape(-1, V)) for i in range(3)]
    wa, wb = oracle(cfg, w, a), oracle(cfg, w, b)
    assert_close(r[0], wa[6:7]); assert_close(r[1], wb[[2, 8]]); assert_close(r[2], wa[11:12])


# -- the HIP path ------------------------------------------------------------------------


@pytest.mark.gpu
@pytest.mark.parametrize("cuts", [[40], [13, 2, 1, 9], []])
def test_gpu_fp32_matches_oracle(cuts):
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=6)
    toks = tokens_of(40, cfg["vocab"], 7)
    eng = engine_for(build(cfg, w, device="cuda"))
    assert_close(run_in_portions(eng, toks, cuts), oracle(cfg, w, toks))


@pytest.mark.gpu
def test_gpu_fp32_mixed_batch_and_reuse():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=12)
    eng = engine_for(build(cfg, w, device="cuda"), pages=9, slots=2)
    for round_ in range(2):                                         # the second round reuses pages and slots
        a, b = tokens_of(30, cfg["vocab"], 60 + round_), tokens_of(11, cfg["vocab"], 70 + round_)
        ra, rb = eng.open_request(), eng.open_request()
        o1 = eng.forward_batch([(ra, a[:17]), (rb, b[:1])], [list(range(17)), [0]])
        o2 = eng.forward_batch([(ra, a[17:18]), (rb, b[1:])], [[0], list(range(10))])
        o3 = eng.forward_batch([(ra, a[18:])], [list(range(12))])
        eng.close_request(ra); eng.close_request(rb)
        assert_close(torch.cat([o1[:17], o2[:1], o3]), oracle(cfg, w, a))
        assert_close(torch.cat([o1[17:], o2[1:]]), oracle(cfg, w, b))


@pytest.mark.gpu
@pytest.mark.parametrize("n,target", [(300, 3), (290, 194), (130, 128), (130, 127)])
@pytest.mark.parametrize("maps", [1, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_far_and_border_keys(n, target, maps, dtype):
    """the planted key on the kernels: fp32 on the VALU, bf16 on the matrix cores (whole tiles and split keys)"""
    from megatron_amd.ops import ragged as R

    H, G, D, V, page = 4, 2, 8, 8, 16
    q, k, v = _planted(n, H, G, maps, D, V, target, 5)
    rep = H // G
    ctx, table, slot = _module_ctx({"c": G * (maps * D + V)}, n, page, dtype=dtype, device="cuda")
    rows = torch.cat([k.reshape(n, -1), v.reshape(n, -1)], dim=1).to(dtype).cuda()
    for cuts in ([n - 1, 1], [n - 40, 40]):
        at = 0
        for c in cuts:
            batch = ctx.begin_batch([c], [at], [slot], [table])
            ctx.pools["c"][batch.tok_row] = rows[at:at + c]
            got = R.map_attention(q[at:at + c].reshape(c, -1).to(dtype).cuda(), ctx.pools["c"], H, G, maps, D, V, 1.0, 0.0,
                                  batch)
            at += c
        last = got[-1].view(H * maps, V).float().cpu()
        own = torch.stack([v[target, qh // (rep * maps)] for qh in range(H * maps)])
        assert (last - own).abs().max().item() < 0.2


@pytest.mark.gpu
def test_gpu_bf16_close_to_oracle():
    """bf16 storage with fp32 residual, norms and scores; routing takes every expert so that rounding
    cannot flip a close choice; head sizes that run on the matrix cores"""
    layers = [att(dim=16, vdim=8, rot=8, experts=3, top=3), att2(heads=2, kv=2, dim=8, vdim=16, rot=4, mlp="dense"),
              att(heads=2, kv=2, dim=8, vdim=8, rot=8, cap=None, mlp="dense"), att2(dim=16, vdim=8, rot=8, mlp="moe", experts=2, top=2)]
    cfg = make_config(layers, width=32)
    w = make_weights(cfg, seed=31)
    toks = tokens_of(44, cfg["vocab"], 32)
    want = oracle(cfg, w, toks)
    eng = engine_for(build(cfg, w, dtype=torch.bfloat16, device="cuda"))
    for cuts in ([44], [9, 2, 20], []):
        got = run_in_portions(eng, toks, cuts).float().cpu()
        d = got - want.float()
        err = (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt() / want.float().std().item()
        assert err.median().item() < 0.03 and err.quantile(0.9).item() < 0.1 and err.max().item() < 0.8, err


@pytest.mark.gpu
def test_gpu_greedy_generation():
    cfg = make_config(FULL)
    w = make_weights(cfg, seed=23)
    prompts = [tokens_of(n, cfg["vocab"], 50 + n) for n in (13, 4, 21)]
    eng = engine_for(build(cfg, w, device="cuda"), pages=16, slots=2, max_prefill_tokens=10)
    res = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=5, stop_on_eod=False))
    for p, r in zip(prompts, res):
        seq = list(p)
        for tok in r.output_tokens:
            logits = oracle(cfg, w, seq)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() > 1e-3:
                assert tok == int(logits.argmax())
            seq.append(tok)
