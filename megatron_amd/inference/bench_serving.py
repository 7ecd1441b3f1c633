"""Serving throughput of ragged-batch models beside the closest existing model.

For each size: random-init weights, bf16, synthetic prompts.  Prefill =
``batch`` prompts of ``isl`` tokens run to their last token; decode = ``osl``
steps of one token per request.  The new design runs through
DynamicInferenceEngine.forward_batch (one mixed forward per step); the
comparison model is GPTModel with multi-latent attention at the same width,
depth, heads and ranks through the same engine class (its paged-latent path:
one prompt per prefill step, batched decode steps).  One JSON line per
(size, model), tokens/s for both phases.

``--serve-design bezurax`` measures the Bezurax design (pooled-window attention
beside a delta-rule memory, routed experts) next to the Bezutar design with
alternating attention / mLSTM layers at the same width, depth and active
feed-forward size, both through the same ragged engine path.

``--serve-design tilarax`` measures the Tilarax design (mLSTM layers alternating
with chunked talking-heads attention layers, post-sublayer norms with a
depth-weighted residual history, dense and routed feed-forwards in turn) next
to the same Bezutar pattern.

``--serve-design lomazen`` measures the Lomazen design (gated capped attention
and differential attention layers with norms on both sides of every sublayer,
a block of layers that runs twice, dense GELU-GLU and routed squared-ReLU
feed-forwards in turn) next to Tilarax with attention layers only
(``tilarax[aA]``: dense and routed feed-forwards in turn) at the same width,
number of layer runs, head sizes and expert sizes.
"""

from __future__ import annotations

import json
import time

import torch

SIZES = {
    # width, layers, heads, qk dim (unrotated), rot, vdim, kv_rank, q_rank, ff, mlstm heads/dim/vdim, mingru width
    "1b": dict(width=2048, layers=8, heads=16, dim=64, rot=32, vdim=64, kv_rank=256, q_rank=768, ff=5632,
               m_heads=4, m_dim=128, m_vdim=256, gru=4096, vocab=32000),
    "7b-layers": dict(width=4096, layers=4, heads=32, dim=128, rot=64, vdim=128, kv_rank=512, q_rank=1536,
                      ff=11008, m_heads=8, m_dim=256, m_vdim=512, gru=8192, vocab=32000),
}


def bezutar_config(s, pattern, max_pos):
    att = dict(type="latent_attention",
               mixer=dict(heads=s["heads"], dim=s["dim"], rot_dim=s["rot"], vdim=s["vdim"], kv_rank=s["kv_rank"],
                          q_rank=s["q_rank"], scale=(s["dim"] + s["rot"]) ** -0.5,
                          rot=dict(base=10000.0, dims=s["rot"],
                                   scaling=dict(factor=4.0, original=max_pos // 4, fast=32.0, slow=1.0))),
               mlp=dict(kind="dense", ff=s["ff"]))
    kinds = {
        "A": att,
        "M": dict(type="mlstm", mixer=dict(heads=s["m_heads"], dim=s["m_dim"], vdim=s["m_vdim"], gate_cap=15.0),
                  mlp=dict(kind="dense", ff=s["ff"])),
        "G": dict(type="mingru", mixer=dict(width=s["gru"]), mlp=dict(kind="dense", ff=s["ff"])),
    }
    layers = [json.loads(json.dumps(kinds[pattern[i % len(pattern)]])) for i in range(s["layers"])]
    return dict(architecture="Bezutar", vocab=s["vocab"], width=s["width"], max_positions=max_pos,
                norm=dict(eps=1e-6), streams=4, canon=dict(taps=4),
                embedding=dict(bigram=dict(buckets=50021, mul_prev=31, mul_cur=17)), layers=layers)


# Bezurax at the same widths and depths: query heads x 128, a quarter as many kv heads,
# window 1024 with 16-token pooled blocks; delta-rule heads of 64; 16 experts of which 3
# are chosen plus a shared one: the active feed-forward size equals the dense ff above
X_SIZES = {
    "1b": dict(heads=16, kv=4, dim=128, window=1024, pool=16, r_heads=16, r_dim=64, experts=16, top=3, eff=1408,
               sff=1408, groups=4, keep=2),
    "7b-layers": dict(heads=32, kv=8, dim=128, window=1024, pool=16, r_heads=32, r_dim=64, experts=16, top=3,
                      eff=2752, sff=2752, groups=4, keep=2),
}


def bezurax_config(size):
    s, x = SIZES[size], X_SIZES[size]
    one = dict(type="parallel",
               mixer=dict(left=dict(heads=x["heads"], kv_heads=x["kv"], dim=x["dim"], vdim=x["dim"],
                                    scale=x["dim"] ** -0.5, mask=dict(size=x["window"], pool=x["pool"])),
                          right=dict(heads=x["r_heads"], dim=x["r_dim"]), left_scale=1.0, right_scale=1.0),
               mlp=dict(kind="moe", expert=dict(ff=x["eff"], limit=7.0),
                        router=dict(experts=x["experts"], top=x["top"], scale=1.0,
                                    groups=dict(count=x["groups"], keep=x["keep"])),
                        shared=dict(ff=x["sff"], limit=7.0)))
    return dict(architecture="Bezurax", vocab=s["vocab"], width=s["width"], norm=dict(eps=1e-6, groups=4),
                logit_scale=1.0, layers=[json.loads(json.dumps(one)) for _ in range(s["layers"])])


# Tilarax at the same widths and depths: mLSTM layers (the sizes above) with a dense feed-forward
# alternate with attention layers of query heads x 128, a quarter as many kv heads, chunks of
# 1024 positions, half of every head rotated, values mixed with the first attention layer's, and
# 16 experts of which 4 are chosen: the active feed-forward size equals the dense ff above
T_SIZES = {
    "1b": dict(heads=16, kv=4, dim=128, chunk=1024, rot=64, experts=16, top=4, eff=1408),
    "7b-layers": dict(heads=32, kv=8, dim=128, chunk=1024, rot=64, experts=16, top=4, eff=2752),
}


def tilarax_config(size, pattern="MA"):
    """pattern, repeated over the depth: M mLSTM + dense, A attention + experts, a attention + dense"""
    s, x = SIZES[size], T_SIZES[size]
    rec = dict(type="mlstm", mixer=dict(heads=s["m_heads"], dim=s["m_dim"], vdim=s["m_vdim"], gate_cap=15.0),
               mlp=dict(kind="dense", ff=s["ff"]))
    att = dict(type="attention",
               mixer=dict(heads=x["heads"], kv_heads=x["kv"], dim=x["dim"], vdim=x["dim"], scale=x["dim"] ** -0.5,
                          mask=dict(size=x["chunk"]), rot=dict(base=10000.0, dims=x["rot"]), v_mix=True),
               mlp=dict(kind="moe", expert=dict(ff=x["eff"]), router=dict(experts=x["experts"], top=x["top"])))
    att_dense = dict(att, mlp=dict(kind="dense", ff=s["ff"]))
    kinds = {"M": rec, "A": att, "a": att_dense}
    layers = [json.loads(json.dumps(kinds[pattern[i % len(pattern)]])) for i in range(s["layers"])]
    return dict(architecture="Tilarax", vocab=s["vocab"], width=s["width"], norm=dict(eps=1e-6), layers=layers)


# Lomazen at the same widths: gated attention layers (query heads x 128, a quarter as many kv heads,
# capped scores, every head rotated with rescaled frequencies) with a dense feed-forward alternate
# with differential attention layers (half as many heads, two maps of 128 each, values of 256, a
# quarter of every map rotated) with 16 experts of which 4 are chosen; the middle layers run twice,
# so that the number of layer runs equals the depth of the comparison
L_SIZES = {
    "1b": dict(layers=6, loop=(2, 4, 2)),
    "7b-layers": dict(layers=3, loop=(1, 2, 2)),
}


def lomazen_config(size):
    s, x, z = SIZES[size], T_SIZES[size], L_SIZES[size]
    one = dict(type="attention",
               mixer=dict(heads=x["heads"], kv_heads=x["kv"], dim=x["dim"], vdim=x["dim"], scale=x["dim"] ** -0.5,
                          softcap=30.0, rot=dict(base=1000000.0, dims=x["dim"],
                                                 scaling=dict(factor=8.0, low=1.0, high=4.0, original=1024))),
               mlp=dict(kind="dense", ff=s["ff"]))
    two = dict(type="attention_2",
               mixer=dict(heads=x["heads"] // 2, kv_heads=max(1, x["kv"] // 2), dim=x["dim"], vdim=2 * x["dim"],
                          scale=x["dim"] ** -0.5, diff=0.5, rot=dict(base=10000.0, dims=x["dim"] // 4)),
               mlp=dict(kind="moe", expert=dict(ff=x["eff"]), router=dict(experts=x["experts"], top=x["top"])))
    layers = [json.loads(json.dumps(two if i % 2 else one)) for i in range(z["layers"])]
    a, b, t = z["loop"]
    assert a + (b - a) * t + (z["layers"] - b) == s["layers"], "layer runs equal the comparison's depth"
    return dict(architecture="Lomazen", vocab=s["vocab"], width=s["width"], norm=dict(eps=1e-6), logit_scale=1.0,
                loop=dict(start=a, stop=b, times=t), layers=layers)


def _random_init(model, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    with torch.no_grad():
        for name, p in model.named_parameters():
            if p.dim() >= 2 and p.dtype != torch.float32:
                fan_in = p.shape[-1]
                p.copy_((torch.randn(p.shape, generator=g) * fan_in ** -0.5).to(p.dtype))
            elif name.endswith(("w_gates", "w_router", "w2")):
                p.copy_(torch.randn(p.shape, generator=g) * p.shape[-1] ** -0.5)
            elif name.endswith("weight") and p.dim() == 2:      # canon taps
                p.copy_(torch.randn(p.shape, generator=g) * 0.2)
            elif name.endswith(".dwa"):                         # mostly the layer's own result
                p.fill_(0.1)
                p[-1] = 1.0
            elif name.endswith(".talk"):
                p.add_((torch.randn(p.shape, generator=g) * 0.1).to(p.device))
            elif name.endswith(".lam"):
                p.fill_(0.3)


def _time(fn):
    sync = torch.cuda.synchronize if torch.cuda.is_available() else (lambda: None)
    sync()
    t0 = time.perf_counter()
    fn()
    sync()
    return time.perf_counter() - t0


def run_bezutar(size, pattern, batch, isl, osl, device):
    from megatron_amd.models.bezutar import BezutarConfig, BezutarModel

    s = SIZES[size]
    cfg = BezutarConfig.from_dict(bezutar_config(s, pattern, isl + osl + 64), dtype=torch.bfloat16)
    with torch.device(device):
        model = BezutarModel(cfg).eval()
    _random_init(model)
    return _run_ragged(model, f"bezutar[{pattern}]", size, batch, isl, osl, device)


def run_bezurax(size, batch, isl, osl, device):
    from megatron_amd.models.bezurax import BezuraxConfig, BezuraxModel

    cfg = BezuraxConfig.from_dict(bezurax_config(size), dtype=torch.bfloat16)
    with torch.device(device):
        model = BezuraxModel(cfg).eval()
    _random_init(model)
    return _run_ragged(model, "bezurax", size, batch, isl, osl, device)


def run_tilarax(size, batch, isl, osl, device, pattern="MA"):
    from megatron_amd.models.tilarax import TilaraxConfig, TilaraxModel

    cfg = TilaraxConfig.from_dict(tilarax_config(size, pattern), dtype=torch.bfloat16)
    with torch.device(device):
        model = TilaraxModel(cfg).eval()
    _random_init(model)
    return _run_ragged(model, "tilarax" if pattern == "MA" else f"tilarax[{pattern}]", size, batch, isl, osl, device)


def run_lomazen(size, batch, isl, osl, device):
    from megatron_amd.models.lomazen import LomazenConfig, LomazenModel

    cfg = LomazenConfig.from_dict(lomazen_config(size), dtype=torch.bfloat16)
    with torch.device(device):
        model = LomazenModel(cfg).eval()
    _random_init(model)
    return _run_ragged(model, "lomazen", size, batch, isl, osl, device)


def _run_ragged(model, label, size, batch, isl, osl, device):
    from megatron_amd.inference.engine import DynamicInferenceEngine

    s = SIZES[size]
    page = 64
    eng = DynamicInferenceEngine(model, num_blocks=batch * ((isl + osl) // page + 2), block_size=page,
                                 max_batch=batch, device=device, use_hip_graphs=False,
                                 enable_prefix_caching=False)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, s["vocab"], (isl,), generator=g).tolist() for _ in range(batch)]

    def once():
        reqs = [eng.open_request() for _ in range(batch)]
        t_pre = _time(lambda: eng.forward_batch([(r, p) for r, p in zip(reqs, prompts)]))
        toks = [[int(x)] for x in torch.randint(0, s["vocab"], (batch,), generator=g)]

        def dec():
            for _ in range(osl):
                eng.forward_batch([(r, t) for r, t in zip(reqs, toks)])
        t_dec = _time(dec)
        for r in reqs:
            eng.close_request(r)
        return t_pre, t_dec

    once()                      # warm-up (GEMM algorithm selection, allocator)
    t_pre, t_dec = once()
    n = sum(p.numel() for p in model.parameters())
    return dict(model=label, size=size, params_m=round(n / 1e6, 1),
                prefill_tok_s=round(batch * isl / t_pre, 1), decode_tok_s=round(batch * osl / t_dec, 1),
                prefill_ms=round(1e3 * t_pre, 2), decode_ms_per_step=round(1e3 * t_dec / osl, 3))


def run_gpt_mla(size, batch, isl, osl, device):
    from megatron_amd.config import TransformerConfig
    from megatron_amd.inference.engine import DynamicInferenceEngine
    from megatron_amd.inference.sampling import SamplingParams
    from megatron_amd.models.gpt import GPTModel
    from megatron_amd.parallel import grid as G
    from megatron_amd.parallel.random import model_parallel_seed

    s = SIZES[size]
    if not G.grid_initialized():
        G.initialize_model_parallel(world_size=1, rank=0)
    model_parallel_seed(1234)
    cfg = TransformerConfig(
        num_layers=s["layers"], hidden_size=s["width"], num_attention_heads=s["heads"],
        ffn_hidden_size=s["ff"], vocab_size=s["vocab"], max_position_embeddings=isl + osl + 64, bf16=True,
        multi_latent_attention=True, q_lora_rank=s["q_rank"], kv_lora_rank=s["kv_rank"],
        qk_nope_head_dim=s["dim"], qk_rope_head_dim=s["rot"], v_head_dim=s["vdim"])
    with torch.device(device):
        model = GPTModel(cfg).eval()
    page = 64
    eng = DynamicInferenceEngine(model, num_blocks=batch * ((isl + osl) // page + 2), block_size=page,
                                 max_batch=batch, max_prefill_tokens=isl, device=device,
                                 use_hip_graphs=False, enable_prefix_caching=False)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, s["vocab"], (isl,), generator=g).tolist() for _ in range(batch)]
    params = SamplingParams(max_tokens=osl + 1, greedy=True, stop_on_eod=False)

    def once():
        for p in prompts:
            eng.add_request(p, params)

        def pre():
            for _ in range(batch):
                eng.step()

        def dec():
            for _ in range(osl):
                eng.step()
        t_pre, t_dec = _time(pre), _time(dec)
        eng.finished.clear()
        assert not eng.has_work()
        return t_pre, t_dec

    once()
    t_pre, t_dec = once()
    n = sum(p.numel() for p in model.parameters())
    return dict(model="gpt-mla", size=size, params_m=round(n / 1e6, 1),
                prefill_tok_s=round(batch * isl / t_pre, 1), decode_tok_s=round(batch * osl / t_dec, 1),
                prefill_ms=round(1e3 * t_pre, 2), decode_ms_per_step=round(1e3 * t_dec / osl, 3))


def main(args) -> None:
    assert torch.cuda.is_available(), "the serving comparison needs a GPU"
    device = torch.device("cuda", 0)
    torch.cuda.set_device(0)
    for size in args.serve_sizes.split(","):
        design = getattr(args, "serve_design", "bezutar")
        if design in ("bezurax", "tilarax"):
            run = run_bezurax if design == "bezurax" else run_tilarax
            r = run(size, args.serve_batch, args.serve_isl, args.serve_osl, device)
            r.update(batch=args.serve_batch, isl=args.serve_isl, osl=args.serve_osl, dtype="bf16", data="synthetic")
            print(json.dumps(r), flush=True)
            torch.cuda.empty_cache()
        if design == "lomazen":
            # the new design, then the closest existing one (attention layers only); no Bezutar patterns
            which = getattr(args, "serve_models", "lomazen,tilarax").split(",")
            for name in which:
                if name == "lomazen":
                    r = run_lomazen(size, args.serve_batch, args.serve_isl, args.serve_osl, device)
                else:
                    r = run_tilarax(size, args.serve_batch, args.serve_isl, args.serve_osl, device, "aA")
                r.update(batch=args.serve_batch, isl=args.serve_isl, osl=args.serve_osl, dtype="bf16", data="synthetic")
                print(json.dumps(r), flush=True)
                torch.cuda.empty_cache()
            continue
        for pattern in [p for p in args.serve_patterns.split(",") if p and p != "none"]:
            r = run_bezutar(size, pattern, args.serve_batch, args.serve_isl, args.serve_osl, device)
            r.update(batch=args.serve_batch, isl=args.serve_isl, osl=args.serve_osl, dtype="bf16", data="synthetic")
            print(json.dumps(r), flush=True)
            torch.cuda.empty_cache()
        if not args.serve_skip_baseline:
            r = run_gpt_mla(size, args.serve_batch, args.serve_isl, args.serve_osl, device)
            r.update(batch=args.serve_batch, isl=args.serve_isl, osl=args.serve_osl, dtype="bf16", data="synthetic")
            print(json.dumps(r), flush=True)
            torch.cuda.empty_cache()
