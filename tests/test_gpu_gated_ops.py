"""GPU numerics of the gated-extension serving kernels (norms on both sides of a
sublayer, restart of a repeated block, rotation in pairs / halves with unit norm
and cache store, attention with one or two softmax maps a head on the VALU and
on the matrix cores with capped scores, gated and differential finish, squared
ReLU, tanh-GELU GLU, the softmax-over-all router, experts without a gate
matrix): every kernel against the plain torch implementation of the same op
(ops/ragged_reference.py) on the same inputs, in fp32 and bf16 storage, on a
ragged batch that mixes prompt portions with single tokens and uses skewed page
tables."""

import pytest
import torch

pytestmark = pytest.mark.gpu

from test_gpu_ragged_ops import _both, _close, _ctx, _rand  # noqa: E402

COUNTS, STARTS = [45, 1, 7, 2, 1], [0, 52, 30, 3, 11]
LONG = [0, 300, 130, 3, 517]


def _need():
    from megatron_amd.ops import ragged as R

    assert R._load("gated") is not None, "gated-ops extension must be built for GPU tests"
    return R


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ydtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [200, 202, 1027, 2048])
def test_sandwich_norm_add_and_restart(dtype, ydtype, W):
    """widths that are and are not a multiple of four, above one pass of a workgroup; a strided copy target"""
    R = _need()
    T = 13

    def run(dev, dt):
        x = _rand((T, W), torch.float32, dev, 2.0)
        outs = []
        wide = torch.zeros(T, 2 * W + 4, dtype=dt, device=dev)
        for k in range(3):
            y = _rand((T, W), ydtype, dev, 3.0)
            wp, wn = _rand((W,), torch.float32, dev), _rand((W,), torch.float32, dev)
            outs.append(R.sandwich_norm_add(x, y, wp, wn, 1e-5, dt).clone())
        outs.append(R.sandwich_norm_add(x, None, None, _rand((W,), torch.float32, dev), 1e-5, dt).clone())
        y = _rand((T, W), ydtype, dev, 0.5)
        assert R.sandwich_norm_add(x, y, _rand((W,), torch.float32, dev), None, 1e-5, dt, copy_to=wide[:, 4:4 + W]) is None
        R.sandwich_norm_add(x, None, None, None, 1e-5, dt, copy_to=wide[:, 4 + W:])
        outs.append(wide.clone())
        x2, h2 = R.restart_norm(_rand((T, W), ydtype, dev), _rand((W,), torch.float32, dev),
                                _rand((W,), torch.float32, dev), 1e-5, dt)
        return outs + [h2, x2, x]

    g, c = _both(run, dtype)
    for i, (a, b) in enumerate(zip(g, c)):
        _close(a, b, dtype if i < len(g) - 2 else torch.float32, f"output {i}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 24, 32, 8), (3, 3, 80, 40, 80), (6, 1, 144, 8, 0), (2, 2, 7, 5, 4),
                                   (8, 2, 64, 64, 32), (5, 5, 130, 12, 130)])
@pytest.mark.parametrize("layout", ["pairs", "halves"])
@pytest.mark.parametrize("unit", [False, True])
def test_rope_norm_store(dtype, shape, layout, unit):
    """q heads, k heads, dim, value width, rotated dims (0: none; an odd head size keeps entries that pass);
    the projection carries extra columns behind the values"""
    R = _need()
    QH, KH, D, VW, rot = shape

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": KH * D + VW}, {}, COUNTS, [0, 52, 30, 3, 1500])
        T = sum(COUNTS)
        proj = _rand((T, (QH + KH) * D + VW + 9), dt, dev)
        freqs = R.scaled_freqs(rot, 5000.0, {"factor": 6.0, "low": 1.5, "high": 5.0, "original": 64}, dev)
        q = R.rope_norm_store(proj, QH, KH, D, VW, freqs, layout, unit, 1e-5, ctx.pools["c"], ctx.batch)
        return q, ctx.pools["c"]

    g, c = _both(run, dtype)
    _close(g[0], c[0], dtype, "q")
    _close(g[1], c[1], dtype, "cache rows")


SHAPES = [(4, 2, 1, 24, 24), (3, 3, 2, 80, 40), (6, 1, 1, 144, 144), (2, 2, 2, 16, 8), (8, 2, 1, 64, 64),
          (2, 1, 1, 12, 20), (4, 4, 2, 32, 48), (1, 1, 1, 256, 256), (8, 4, 1, 40, 88), (4, 2, 2, 56, 104),
          (2, 2, 2, 160, 128), (16, 8, 1, 128, 128), (4, 1, 2, 128, 256)]


@pytest.fixture(params=[(torch.float32, 64), (torch.bfloat16, 64), (torch.bfloat16, 128)],
                ids=["float32", "bfloat16-rows64", "bfloat16-rows128"])
def dtype_tiles(request, monkeypatch):
    """fp32 (VALU kernel) and bf16 with both tile sizes of the matrix-core kernel, whatever the step's
    size would choose; -> the storage dtype"""
    monkeypatch.setenv("MEGATRON_AMD_MAP_TILE_ROWS", str(request.param[1]))
    return request.param[0]


@pytest.mark.parametrize("shape", SHAPES + [(6, 3, 1, 40, 72), (2, 2, 2, 200, 136)])
@pytest.mark.parametrize("starts", [STARTS, LONG], ids=["short", "long"])
@pytest.mark.parametrize("cap", [0.0, 3.0])
def test_map_attention(dtype_tiles, shape, starts, cap):
    """heads, kv heads, maps, dim, vdim; page 16; long contexts beside short ones make the bf16 kernel
    split the key tiles; the shapes cover every matrix-core instantiation and sizes it does not take"""
    R = _need()
    dtype = dtype_tiles
    H, G, M, D, V = shape

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": G * (M * D + V)}, {}, COUNTS, starts)
        pool = ctx.pools["c"]
        pool.copy_(_rand(pool.shape, dt, dev))            # what earlier steps left (and junk in foreign pages)
        q = _rand((sum(COUNTS), H * M * D), dt, dev)
        return R.map_attention(q, pool, H, G, M, D, V, 2.0 * D ** -0.5, cap, ctx.batch)

    g, c = _both(run, dtype)
    _close(g, c, dtype, "attention")


@pytest.mark.parametrize("shape", [s for s in SHAPES if s[2] == 1])
@pytest.mark.parametrize("starts", [STARTS, LONG], ids=["short", "long"])
def test_softcap_gated_attention(dtype_tiles, shape, starts):
    """the gate is a strided view behind other columns, as a fused projection's slice is"""
    R = _need()
    dtype = dtype_tiles
    H, G, _, D, V = shape

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": G * (D + V)}, {}, COUNTS, starts)
        pool = ctx.pools["c"]
        pool.copy_(_rand(pool.shape, dt, dev))
        T = sum(COUNTS)
        q = _rand((T, H * D), dt, dev)
        wide = _rand((T, 7 + H * V), dt, dev)
        return R.softcap_gated_attention(q, wide[:, 7:], pool, H, G, D, V, D ** -0.5, 5.0, ctx.batch)

    g, c = _both(run, dtype)
    _close(g, c, dtype, "gated attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [s for s in SHAPES if s[2] == 2])
@pytest.mark.parametrize("starts", [STARTS, LONG], ids=["short", "long"])
def test_differential_attention(dtype, shape, starts):
    R = _need()
    H, G, _, D, V = shape

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": G * (2 * D + V)}, {}, COUNTS, starts)
        pool = ctx.pools["c"]
        pool.copy_(_rand(pool.shape, dt, dev))
        T = sum(COUNTS)
        q = _rand((T, H * 2 * D), dt, dev)
        wide = _rand((T, 3 + H), dt, dev)
        lam = torch.tensor([0.7], device=dev)
        return R.differential_attention(q, wide[:, 3:], lam, 0.4, 1e-5, pool, H, G, D, V, D ** -0.5, ctx.batch)

    g, c = _both(run, dtype)
    _close(g, c, dtype, "differential attention")


def test_map_attention_prompt_tiles(dtype_tiles):
    """long portions: several row tiles per request; rows of one tile end in different key tiles; a last
    tile whose later row tiles are empty; a first row tile that ends before the key tile the second needs"""
    R = _need()
    dtype = dtype_tiles
    H, G, M, D, V = 4, 2, 2, 64, 32

    def run(dev, dt):
        ctx = _ctx(dev, dt, {"c": G * (M * D + V)}, {}, [150, 1, 90, 40], [0, 99, 37, 24])
        pool = ctx.pools["c"]
        pool.copy_(_rand(pool.shape, dt, dev))
        q = _rand((281, H * M * D), dt, dev)
        return R.map_attention(q, pool, H, G, M, D, V, 0.2, 0.0, ctx.batch)

    g, c = _both(run, dtype)
    _close(g, c, dtype, "attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_relu2_and_gelu_glu(dtype):
    R = _need()

    def run(dev, dt):
        z = _rand((37, 130), dt, dev, 2.0)
        return R.relu2(z, dt), R.glu(z, "gelu_tanh", 0.0, 0.0, dt), R.relu2(z[:, :129].contiguous(), dt)

    g, c = _both(run, dtype)
    for a, b, n in zip(g, c, ["relu2", "gelu glu", "relu2, odd count"]):
        _close(a, b, dtype, n)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("top", [1, 4, 10])
def test_softmax_all_router_and_plain_pairs(dtype, top):
    R = _need()
    E, W, F_ = 10, 64, 24

    def run(dev, dt):
        h = _rand((5, W), dt, dev)
        wr = _rand((E, W), torch.float32, dev)
        ids, wts, extra = R.moe_router(h, wr, E, top, 1, 1, 1.0, None, "softmax_all")
        wu, wd = _rand((E, F_, W), dt, dev, 0.2), _rand((E, W, F_), dt, dev, 0.2)
        down = R.expert_pairs_plain(h, ids, wu, wd)
        return ids.float(), wts, down

    g, c = _both(run, dtype)
    assert torch.equal(g[0].cpu(), c[0]), "chosen experts"
    _close(g[1], c[1], torch.float32, "weights")
    _close(g[2], c[2], dtype, "pair outputs")
