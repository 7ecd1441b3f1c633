"""GPU numerics of the talking-heads serving kernels (post-sublayer norm with a
depth-weighted residual history, per-head q/k norm with pairwise rotation and
value mixing, chunked talking-heads attention on the VALU and on the matrix
cores, tanh-GELU, the softmax-over-chosen router, SiLU-GLU experts): every
kernel against the plain torch implementation of the same op
(ops/ragged_reference.py) on the same inputs, in fp32 and bf16 storage, on a
ragged batch that mixes prompt portions with single tokens, uses skewed page
tables and reused state slots."""

import pytest
import torch

pytestmark = pytest.mark.gpu

from test_gpu_ragged_ops import _both, _close, _ctx, _rand  # noqa: E402

COUNTS, STARTS = [45, 1, 7, 2, 1], [0, 52, 30, 3, 11]


def _need():
    from megatron_amd.ops import ragged as R

    assert R._load("talking") is not None, "talking-ops extension must be built for GPU tests"
    return R


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ydtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [200, 202, 1027])
def test_post_norm_add_and_depth_history(dtype, ydtype, W):
    """widths that are and are not a multiple of four (the kernel's wide accesses), above one pass of a workgroup"""
    R = _need()
    T, L = 13, 3

    def run(dev, dt):
        x = _rand((T, W), torch.float32, dev)
        hist = torch.zeros(L + 1, T, W, device=dev)
        hist[0].copy_(x)
        outs = []
        for depth in range(1, L + 1):
            y = _rand((T, W), ydtype, dev, 3.0)
            w = _rand((W,), torch.float32, dev, 0.2)
            outs.append(R.post_norm_add(x, y, w, 1e-5, dt).clone())
            y2 = _rand((T, W), ydtype, dev, 0.3)
            dwa = _rand((depth + 1,), torch.float32, dev)
            outs.append(R.post_norm_add(x, y2, w, 1e-5, dt, hist, depth, dwa).clone())
        outs.append(R.post_norm_add(x, None, None, 1e-5, dt, hist, L, _rand((L + 1,), torch.float32, dev)).clone())
        return outs + [x, hist]

    g, c = _both(run, dtype)
    for i, (a, b) in enumerate(zip(g, c)):
        _close(a, b, dtype if i < len(g) - 2 else torch.float32, f"output {i}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 24, 16, 8), (3, 3, 80, 40, 80), (6, 1, 144, 8, 0), (2, 2, 7, 5, 4),
                                   (8, 2, 64, 64, 32)])
@pytest.mark.parametrize("mix", [False, True])
def test_head_norm_rope_store(dtype, shape, mix):
    """heads, kv heads, dim, vdim, rotated dims (0: none; an odd head size keeps its last entry unpaired)"""
    R = _need()
    H, G, D, V, rot = shape

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": G * (D + V)}, {}, COUNTS, [0, 52, 30, 3, 1500])
        T = sum(COUNTS)
        proj = _rand((T, (H + G) * D + G * V), dt, dev)
        wide = _rand((T, 3 * G * V), dt, dev)
        v_first = wide[:, G * V:2 * G * V] if mix else None       # a strided view, as a projection's slice is
        lam = torch.tensor([0.3], device=dev)
        freqs = R.pair_freqs(rot, 5000.0, dev)
        q = R.head_norm_rope_store(proj, H, G, D, V, _rand((D,), torch.float32, dev), _rand((D,), torch.float32, dev),
                                   1e-5, freqs, v_first, lam, ctx.pools["c"], ctx.batch)
        return q, ctx.pools["c"]

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "q")
    _close(g[1], c[1], dtype, "cache rows")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 24, 24, 9), (3, 3, 80, 40, 0), (6, 1, 144, 144, 64), (2, 2, 16, 8, 1),
                                   (8, 2, 64, 64, 40), (2, 1, 12, 20, 5), (4, 4, 32, 48, 200), (1, 1, 256, 256, 33),
                                   (8, 4, 32, 64, 40), (3, 3, 16, 200, 30), (2, 2, 160, 128, 50), (16, 8, 128, 128, 100)])
@pytest.mark.parametrize("starts", [STARTS, [0, 300, 130, 3, 517]], ids=["short", "long"])
def test_talking_attention(dtype, shape, starts):
    """heads, kv heads, dim, vdim, chunk (0: none); page 16: chunks cross pages and page borders
    lie inside chunks; long contexts beside short ones make the bf16 kernel split the key tiles; the
    last shapes make a workgroup take several value heads, an uneven last group, and wide keys"""
    R = _need()
    H, G, D, V, chunk = shape

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": G * (D + V)}, {}, COUNTS, starts)
        pool = ctx.pools["c"]
        pool.copy_(_rand(pool.shape, dt, dev))            # what earlier steps left (and junk in foreign pages)
        q = _rand((sum(COUNTS), H * D), dt, dev)
        temp = _rand((H,), torch.float32, dev).abs() + 0.5
        talk = _rand((H, H), torch.float32, dev)
        return R.talking_attention(q, pool, H, G, D, V, D ** -0.5, temp, talk, chunk, ctx.batch, dt)

    g, c = _both(run, dtype)
    _close(g, c, dtype, "attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_talking_attention_prompt_tiles(dtype):
    """a long portion: several 64-row tiles per request, rows of a tile in different chunks"""
    R = _need()
    H, G, D, V, chunk = 4, 2, 64, 32, 50

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": G * (D + V)}, {}, [150, 1, 90], [0, 99, 37])
        pool = ctx.pools["c"]
        pool.copy_(_rand(pool.shape, dt, dev))
        q = _rand((241, H * D), dt, dev)
        return R.talking_attention(q, pool, H, G, D, V, 0.2, torch.ones(H, device=dev), _rand((H, H), torch.float32, dev),
                                   chunk, ctx.batch, dt)

    g, c = _both(run, dtype)
    _close(g, c, dtype, "attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu_tanh_and_silu_glu(dtype):
    R = _need()

    def run(dev, dt):
        z = _rand((37, 130), dt, dev, 2.0)
        return R.gelu_tanh(z, dt), R.glu(z, "silu", 0.0, 1.0, dt), R.glu(z, "clamped", 1.5, 1.702, dt)

    g, c = _both(run, dtype)
    for a, b, n in zip(g, c, ["gelu", "silu glu", "clamped glu"]):
        _close(a, b, dtype, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("top", [1, 3, 8])
def test_softmax_router_and_silu_pairs(dtype, top):
    R = _need()
    E, W, F_ = 8, 64, 24

    def run(dev, dt):
        h = _rand((5, W), dt, dev)
        wr, br = _rand((E, W), torch.float32, dev), _rand((E,), torch.float32, dev, 2.0)
        ids, wts, extra = R.moe_router(h, wr, E, top, 1, 1, 1.0, br, "softmax")
        wgu, wd = _rand((E, 2 * F_, W), dt, dev, 0.2), _rand((E, W, F_), dt, dev, 0.2)
        down = R.expert_pairs(h, ids, wgu, wd, 0.0, 1.0, "silu")
        return ids.float(), wts, down

    g, c = _both(run, dtype)
    assert torch.equal(g[0].cpu(), c[0]), "chosen experts"
    _close(g[1], c[1], torch.float32, "weights")
    _close(g[2], c[2], dtype, "pair outputs")
