"""Ragged-batch sequence ops.

``_ragged_ops``: embedding with hashed bigrams, hyper-connection stream mixing
fused with RMS norm, residual causal convolution with carried taps, minGRU and
mLSTM recurrences with per-request state slots, latent-cache attention with a
softmax sink, xIELU.
``_hybrid_ops``: embedding into a plain fp32 residual, residual add fused with
grouped RMS norm, whole-projection q/k norm with cache store, pooled-block
completion and attention over a sliding window plus pooled blocks, generalized
delta rule, expert routing, clamped GLU, pair-streaming experts, expert combine.
``_talking_ops``: post-sublayer norm with a depth-weighted residual history,
per-head q/k norm with pairwise rotation, value mixing and cache store, chunked
talking-heads attention, tanh-GELU; it also carries the embedding, mLSTM and
routed-expert kernels of the other two (same sources), so that a model built
on it compiles nothing else.
``_gated_ops``: norms on both sides of a sublayer, restart of a repeated block
of layers, rotation in pairs or halves with an optional unit norm and cache
store, attention with one or two softmax maps a head (capped scores; gated or
differential finish), squared ReLU, experts without a gate matrix; it carries
the embedding, final-norm, router, GLU and expert kernels of ``_hybrid_ops``
(same sources).

Dispatch rule (same as megatron_amd.ops): tensors on a HIP device run the
CDNA4 kernels of the extension (csrc/ragged/*.hip, csrc/hybrid/*.hip) and RAISE
when it is not built; CPU tensors run the torch implementations in
``ragged_reference`` so every path tests without a GPU.
MEGATRON_AMD_FORCE_REFERENCE=1 forces the torch path (numerics tests).
"""

from __future__ import annotations

import os
from typing import Optional

import torch

from megatron_amd.ops import ragged_reference as ref
from megatron_amd.ops.ragged_reference import rope_table  # noqa: F401  (host-side table)

_C = None      # _ragged_ops: latent attention, mLSTM, minGRU, hyper-connections, canon conv, xIELU
_H = None      # _hybrid_ops: grouped norm, pooled-window attention, delta rule, routed experts
_K = None      # _talking_ops: post-norm with depth history, talking-heads attention (+ shared kernels)
_G = None      # _gated_ops: sandwich norms, capped / differential attention (+ shared kernels)
_IMPORT_ERROR: Optional[str] = None
_IMPORT_ERRORS = {}

# setup.py extension key -> module name; a model names the keys it needs in
# ``native_extensions`` and a serving process builds only those on first use
EXTENSIONS = {"ragged": "_ragged_ops", "hybrid": "_hybrid_ops", "talking": "_talking_ops", "gated": "_gated_ops"}


def _load(key: str = "ragged"):
    global _C, _H, _K, _G, _IMPORT_ERROR
    cur = {"ragged": _C, "hybrid": _H, "talking": _K, "gated": _G}[key]
    if cur is not None:
        return cur
    try:
        import importlib

        mod = importlib.import_module("megatron_amd.ops." + EXTENSIONS[key])  # built in-tree (setup.py)
        if key == "ragged":
            _C = mod
        elif key == "hybrid":
            _H = mod
        elif key == "talking":
            _K = mod
        else:
            _G = mod
        return mod
    except Exception as e:  # noqa: BLE001
        _IMPORT_ERRORS[key] = repr(e)
        if key == "ragged":
            _IMPORT_ERROR = repr(e)
    return None


_load("ragged")
_load("hybrid")
_load("talking")
_load("gated")


def build_extension(key: str, verbose: bool = False) -> None:
    """Compile ONE serving extension in-tree (a serving process of a model that
    needs nothing else calls this on first use)."""
    import subprocess
    import sys

    repo = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env = dict(os.environ, MEGATRON_AMD_ONLY_EXT=key, PYTORCH_ROCM_ARCH="gfx950")
    env.setdefault("MAX_JOBS", "8")
    out = None if verbose else subprocess.DEVNULL
    subprocess.run([sys.executable, "setup.py", "build_ext", "--inplace"], cwd=repo, env=env,
                   check=True, stdout=sys.stderr if verbose else out, stderr=sys.stderr if verbose else out)
    if _load(key) is None:
        raise RuntimeError(f"{EXTENSIONS[key]} did not import after build: {_IMPORT_ERRORS.get(key)}")


def build_ragged_ops(verbose: bool = False) -> None:
    build_extension("ragged", verbose)


def ensure_built(keys, verbose: bool = False) -> None:
    """Build the named extensions that are not there yet."""
    for key in keys:
        if _load(key) is None:
            build_extension(key, verbose)


def has_native() -> bool:
    return _C is not None and os.environ.get("MEGATRON_AMD_FORCE_REFERENCE", "0") != "1"


def _native(x: torch.Tensor) -> bool:
    if not x.is_cuda:
        return False
    if os.environ.get("MEGATRON_AMD_FORCE_REFERENCE", "0") == "1":
        return False
    if _C is None:
        raise RuntimeError(
            "megatron_amd ragged-ops HIP extension not built but a GPU tensor hit the ops layer "
            f"(import error: {_IMPORT_ERROR}). Run megatron_amd.ops.ragged.build_ragged_ops().")
    return True


def _native_h(x: torch.Tensor) -> bool:
    if not x.is_cuda or os.environ.get("MEGATRON_AMD_FORCE_REFERENCE", "0") == "1":
        return False
    if _H is None:
        raise RuntimeError(
            "megatron_amd hybrid-ops HIP extension not built but a GPU tensor hit the ops layer "
            f"(import error: {_IMPORT_ERRORS.get('hybrid')}). Run megatron_amd.ops.ragged.build_extension('hybrid').")
    return True


def _pick(x: torch.Tensor, *keys):
    """The first built extension among ``keys`` for a GPU tensor (several
    extensions carry the same kernel), None for the torch path; raises when a
    GPU tensor finds none of them."""
    if not x.is_cuda or os.environ.get("MEGATRON_AMD_FORCE_REFERENCE", "0") == "1":
        return None
    for key in keys:
        mod = {"ragged": _C, "hybrid": _H, "talking": _K, "gated": _G}[key]
        if mod is not None:
            return mod
    raise RuntimeError(
        f"none of the HIP extensions {keys} is built but a GPU tensor hit the ops layer "
        f"(import errors: {_IMPORT_ERRORS}). Run megatron_amd.ops.ragged.build_extension('{keys[0]}').")


_EMPTY = {}


def _none(device):
    t = _EMPTY.get(device)
    if t is None:
        t = _EMPTY[device] = torch.empty(0, device=device)
    return t


def embed_tokens(tokens, batch, embed, bigram, pos, prev_state, mul_prev=0, mul_cur=0, buckets=1):
    if _native(embed):
        d = embed.device
        return _C.embed_tokens(tokens, batch.cu_tokens, batch.slots, batch.tok_req, batch.tok_pos,
                               embed, bigram if bigram is not None else _none(d),
                               pos if pos is not None else _none(d),
                               prev_state if prev_state is not None else _none(d),
                               int(mul_prev), int(mul_cur), int(buckets))
    return ref.embed_tokens(tokens, batch, embed, bigram, pos, prev_state, mul_prev, mul_cur, buckets)


def hc_mix_norm(streams, y, mix, out_w, in_w, norm_w, eps):
    if _native(streams):
        d = streams.device
        h = _C.hc_mix_norm(streams, y if y is not None else _none(d),
                           mix if y is not None else _none(d), out_w if y is not None else _none(d),
                           in_w if in_w is not None else _none(d),
                           norm_w if in_w is not None else _none(d), float(eps))
        return h if in_w is not None else None
    return ref.hc_mix_norm(streams, y, mix, out_w, in_w, norm_w, eps)


def canon_conv(h, weight, state, batch, out_dtype):
    if _native(h):
        return _C.canon_conv(h, weight, state, batch.cu_tokens, batch.slots, batch.tok_req,
                             out_dtype == torch.bfloat16)
    return ref.canon_conv(h, weight, state, batch, out_dtype)


def mingru_scan(zxg, bias_z, bias_x, state, batch, out_dtype):
    if _native(zxg):
        return _C.mingru_scan(zxg, bias_z, bias_x, state, batch.cu_tokens, batch.slots)
    return ref.mingru_scan(zxg, bias_z, bias_x, state, batch, out_dtype)


def mlstm_scan(qkvg, gates, bias_i, bias_f, norm_w, heads, dim, vdim, cap, eps,
               state_S, state_n, state_m, batch, out_dtype):
    ext = _pick(qkvg, "ragged", "talking")
    if ext is not None:
        return ext.mlstm_scan(qkvg, gates, bias_i, bias_f, norm_w, heads, dim, vdim, float(cap), float(eps),
                             state_S, state_n, state_m, batch.cu_tokens, batch.slots)
    return ref.mlstm_scan(qkvg, gates, bias_i, bias_f, norm_w, heads, dim, vdim, cap, eps,
                          state_S, state_n, state_m, batch, out_dtype)


def latent_kv_store(dkv, norm_w, eps, cos, sin, rot_dims, rank, pool, batch):
    if _native(dkv):
        _C.latent_kv_store(dkv, norm_w, float(eps), cos, sin, int(rot_dims), int(rank), pool,
                           batch.tok_pos, batch.tok_row)
        return
    ref.latent_kv_store(dkv, norm_w, eps, cos, sin, rot_dims, rank, pool, batch)


def latent_q_prepare(dq, norm_w, eps, out_dtype):
    if _native(dq):
        return _C.rmsnorm_rows(dq, norm_w, float(eps))
    return ref.latent_q_prepare(dq, norm_w, eps, out_dtype)


def assemble_latent_q(q_abs, q_rot, cos, sin, rot_dims, batch):
    """[absorbed unrotated part | rotated part after RoPE] -> [T, H, rank + rot]."""
    if _native(q_abs):
        return _C.assemble_latent_q(q_abs, q_rot, cos, sin, int(rot_dims), batch.tok_pos)
    return torch.cat([q_abs, ref.rope_heads(q_rot, cos, sin, rot_dims, batch)], dim=-1)


def _mfma_ok(q, rank) -> bool:
    Dk = q.shape[2]
    return (q.dtype == torch.bfloat16 and Dk % 8 == 0 and rank % 4 == 0 and Dk <= 576 and rank <= 512
            and os.environ.get("MEGATRON_AMD_NO_MFMA_LATENT", "0") != "1")


def latent_sink_attention(q, pool, rank, sink, scale, batch):
    """[T, H, rank] (a view of an [H, T, rank] buffer on the kernel paths)."""
    if _native(q):
        if _mfma_ok(q, rank):
            # matrix-core kernel: 64 (token, head) rows per workgroup; steps with few
            # rows and long contexts (decode) also split the keys over workgroups
            tiles = batch.row_tiles(q.shape[1], q.device)
            nblk = tiles.shape[0]
            nsplit = max(1, min((batch.max_context + 63) // 64, 1024 // nblk, 64))
            return _C.latent_sink_attention_mfma(q, pool, int(rank), sink, float(scale), tiles, batch.cu_tokens,
                                                 batch.start_pos, batch.block_tables, int(batch.block_size),
                                                 int(nsplit))
        return _C.latent_sink_attention(q, pool, int(rank), sink, float(scale), batch.tok_req,
                                        batch.tok_pos, batch.block_tables, int(batch.block_size))
    return ref.latent_sink_attention(q, pool, rank, sink, scale, batch)


def xielu(z, act, out_dtype):
    if _native(z):
        return _C.xielu(z, act)
    return ref.xielu(z, act, out_dtype)


def gate_heads(x, gate_pre, heads):
    if _native(x):
        return _C.gate_heads(x, gate_pre, int(heads))
    return ref.gate_heads(x, gate_pre, heads)


# ---------------------------------------------------------------------------
# ops of the hybrid extension: plain fp32 residual with grouped RMS norm,
# attention over a sliding window plus mean-pooled blocks, generalized delta
# rule, routed clamped-GLU experts
# ---------------------------------------------------------------------------


def embed_plain(tokens, embed):
    ext = _pick(embed, "hybrid", "talking", "gated")
    if ext is not None:
        return ext.embed_plain(tokens, embed)
    return ref.embed_plain(tokens, embed)


def residual_group_norm(x, y, w_a, w_b, groups, eps, out_dtype):
    """x fp32 [T, W] += y in place (y may be None); -> (norm(x) w_a, norm(x) w_b or None)."""
    ext = _pick(x, "hybrid", "talking", "gated")
    if ext is not None:
        d = x.device
        h_a, h_b = ext.residual_group_norm(x, y if y is not None else _none(d), w_a,
                                          w_b if w_b is not None else _none(d), int(groups), float(eps),
                                          out_dtype == torch.bfloat16)
        return h_a, (h_b if w_b is not None else None)
    return ref.residual_group_norm(x, y, w_a, w_b, groups, eps, out_dtype)


def qk_norm_store(proj, q_off, q_width, k_off, k_width, v_off, v_width, q_norm, k_norm, eps, pool, batch):
    if _native_h(proj):
        return _H.qk_norm_store(proj, int(q_off), int(q_width), int(k_off), int(k_width), int(v_off), int(v_width),
                                q_norm, k_norm, float(eps), pool, batch.tok_row)
    return ref.qk_norm_store(proj, q_off, q_width, k_off, k_width, v_off, v_width, q_norm, k_norm, eps, pool, batch)


def pool_blocks(pool, pooled, block, pooled_per_page, batch):
    if _native_h(pool):
        _H.pool_blocks(pool, pooled, int(block), int(pooled_per_page), batch.cu_tokens, batch.start_pos,
                       batch.block_tables, int(batch.block_size), int(batch.max_new))
        return
    ref.pool_blocks(pool, pooled, block, pooled_per_page, batch)


def pooled_window_attention(q, pool, pooled, heads, kv_heads, dim, vdim, scale, window, block,
                            pooled_per_page, batch, out, out_col, out_scale):
    if _native_h(q):
        if (q.dtype == torch.bfloat16 and dim % 8 == 0 and vdim % 8 == 0 and dim <= 256 and vdim <= 256
                and os.environ.get("MEGATRON_AMD_NO_MFMA_WINDOW", "0") != "1"):
            # matrix-core kernel: 64 (token, head-in-group) rows per workgroup and kv head; steps
            # with few rows (decode) also split the key tiles over workgroups
            tiles = batch.row_tiles(heads // kv_heads, q.device)
            nblk = tiles.shape[0] * kv_heads
            keys = min(batch.max_context, window + 64 + batch.max_context // block)
            nsplit = max(1, min((keys + 63) // 64, 1024 // max(nblk, 1), 64))
            _H.pooled_window_attention_mfma(q, pool, pooled, int(heads), int(kv_heads), int(dim), int(vdim),
                                            float(scale), int(window), int(block), int(pooled_per_page), tiles,
                                            batch.cu_tokens, batch.start_pos, batch.block_tables,
                                            int(batch.block_size), int(nsplit), out, int(out_col), float(out_scale))
            return
        _H.pooled_window_attention(q, pool, pooled, int(heads), int(kv_heads), int(dim), int(vdim), float(scale),
                                   int(window), int(block), int(pooled_per_page), batch.tok_req, batch.tok_pos,
                                   batch.block_tables, int(batch.block_size), out, int(out_col), float(out_scale))
        return
    ref.pooled_window_attention(q, pool, pooled, heads, kv_heads, dim, vdim, scale, window, block,
                                pooled_per_page, batch, out, out_col, out_scale)


def delta_rule_scan(proj, r_off, k_off, v_off, g_off, a_off, w_off, w_rank, w2, w0, a_bias, norm_w,
                    heads, dim, eps, state, batch, out, out_col, out_scale):
    if _native_h(proj):
        _H.delta_rule_scan(proj, int(r_off), int(k_off), int(v_off), int(g_off), int(a_off), int(w_off),
                           int(w_rank), w2, w0, a_bias, norm_w, int(heads), int(dim), float(eps), state,
                           batch.cu_tokens, batch.slots, out, int(out_col), float(out_scale))
        return
    ref.delta_rule_scan(proj, r_off, k_off, v_off, g_off, a_off, w_off, w_rank, w2, w0, a_bias, norm_w,
                        heads, dim, eps, state, batch, out, out_col, out_scale)


def moe_route(logits, experts, top, groups, keep, scale):
    if _native_h(logits):
        return _H.moe_route(logits, int(experts), int(top), int(groups), int(keep), float(scale))
    return ref.moe_route(logits, experts, top, groups, keep, scale)


GLU_KINDS = {"clamped": 0, "silu": 1, "gelu_tanh": 2}


def clamped_glu(gu, limit, alpha, out_dtype):
    return glu(gu, "clamped", limit, alpha, out_dtype)


def glu(gu, act, limit, alpha, out_dtype):
    """gu [N, 2F] = [gate | up] -> [N, F]: "clamped": min(g, limit) sigmoid(alpha g) (clamp(u) + 1);
    "silu": g sigmoid(g) u; "gelu_tanh": gelu_tanh(g) u."""
    ext = _pick(gu, "hybrid", "talking", "gated")
    if ext is not None:
        return ext.clamped_glu(gu, float(limit), float(alpha), GLU_KINDS[act])
    if act == "silu":
        return ref.silu_glu(gu, out_dtype)
    if act == "gelu_tanh":
        return ref.gelu_glu(gu, out_dtype)
    return ref.clamped_glu(gu, limit, alpha, out_dtype)


def moe_combine(down, inv, weights, shared, shared_gate, add):
    ext = _pick(down, "hybrid", "talking", "gated")
    if ext is not None:
        d = down.device
        return ext.moe_combine(down, inv, weights, shared if shared is not None else _none(d),
                               shared_gate if shared is not None else _none(d),
                               add if add is not None else _none(d))
    return ref.moe_combine(down, inv, weights, shared, shared_gate, add)


PAIR_PATH_MAX = 32      # (token, choice) pairs up to which every pair streams its expert's matrices itself


def expert_pairs_ok(h, top, ff) -> bool:
    """Steps with few pairs (decoding) skip the sort by expert: see csrc/hybrid/experts.hip."""
    return (h.is_cuda and (_H is not None or _K is not None or _G is not None)
            and os.environ.get("MEGATRON_AMD_FORCE_REFERENCE", "0") != "1"
            and h.shape[0] * top <= PAIR_PATH_MAX and h.shape[1] % 8 == 0 and ff % 8 == 0
            and max(h.shape[1], ff) <= 15360)


def expert_pairs(h, ids, w_gate_up, w_down, limit, alpha, act="clamped"):
    ext = _pick(h, "hybrid", "talking", "gated")
    if ext is not None:
        return ext.expert_pairs(h, ids, w_gate_up, w_down, float(limit), float(alpha), GLU_KINDS[act])
    return ref.expert_pairs(h, ids, w_gate_up, w_down, limit, alpha, act)


ROUTER_SCORES = {"sigmoid": 0, "softmax": 1, "softmax_all": 2}


def moe_router(h, w_router, experts, top, groups, keep, scale, bias=None, score="sigmoid"):
    """-> (ids [T, top] int32, weights [T, top] fp32, raw logits of the rows beyond the experts)

    score "sigmoid": sigmoid scores, group-limited choice, weights = chosen scores / their sum * scale;
    score "softmax": the largest logits are chosen, weights = softmax over the chosen logits;
    score "softmax_all": the largest logits are chosen, weights = their softmax over ALL experts."""
    ext = _pick(h, "hybrid", "talking", "gated")
    if ext is not None and h.shape[1] <= 15360 and w_router.shape[0] <= 512 and top <= 16 and groups <= 64:
        return ext.moe_router(h, w_router, bias if bias is not None else _none(h.device), int(experts), int(top),
                              int(groups), int(keep), float(scale), ROUTER_SCORES[score])
    return ref.moe_router(h, w_router, experts, top, groups, keep, scale, bias, score)


# ---------------------------------------------------------------------------
# ops of the talking extension: post-sublayer norm with a depth-weighted
# residual history, per-head q/k norm with pairwise rotation and value mixing,
# chunked talking-heads attention, tanh-GELU
# ---------------------------------------------------------------------------

pair_freqs = ref.pair_freqs


def _native_k(x: torch.Tensor) -> bool:
    return _pick(x, "talking") is not None


def post_norm_add(x, y, w, eps, out_dtype, hist=None, depth=0, dwa=None):
    """x fp32 [T, W] <- x + rms(y) (1 + w) in place (y may be None); with ``hist``:
    hist[depth] <- x, x <- sum_{j <= depth} dwa[j] hist[j].  -> x in out_dtype."""
    if _native_k(x):
        d = x.device
        return _K.post_norm_add(x, y if y is not None else _none(d), w if y is not None else _none(d), float(eps),
                                out_dtype == torch.bfloat16, hist if hist is not None else _none(d), int(depth),
                                dwa if hist is not None else _none(d))
    return ref.post_norm_add(x, y, w, eps, out_dtype, hist, depth, dwa)


def head_norm_rope_store(proj, heads, kv_heads, dim, vdim, q_norm, k_norm, eps, freqs, v_first, lam, pool, batch):
    if _native_k(proj):
        d = proj.device
        return _K.head_norm_rope_store(proj, int(heads), int(kv_heads), int(dim), int(vdim), q_norm, k_norm,
                                       float(eps), freqs, v_first if v_first is not None else _none(d),
                                       lam if v_first is not None else _none(d), pool, batch.tok_pos, batch.tok_row)
    return ref.head_norm_rope_store(proj, heads, kv_heads, dim, vdim, q_norm, k_norm, eps, freqs, v_first, lam,
                                    pool, batch)


def talking_attention(q, pool, heads, kv_heads, dim, vdim, scale, temp, talk, chunk, batch, out_dtype):
    """-> [T, heads * vdim] in out_dtype"""
    if _native_k(q):
        if (q.dtype == torch.bfloat16 and dim % 8 == 0 and vdim % 8 == 0 and dim <= 256 and vdim <= 256
                and os.environ.get("MEGATRON_AMD_NO_MFMA_TALKING", "0") != "1"):
            # matrix-core kernel: 64 (token, head-in-group) rows per workgroup and (key head, group of
            # value heads) pair; steps with few rows (decode) also split the key tiles over workgroups
            tiles = batch.row_tiles(heads // kv_heads, q.device)
            groups = max(1, (kv_heads * vdim + 511) // 512)
            if tiles.shape[0] * kv_heads * groups < 256:      # the kernel's rule: one value head a workgroup
                groups = kv_heads
            nblk = tiles.shape[0] * kv_heads * groups
            keys = min(batch.max_context, chunk) if chunk > 0 else batch.max_context
            nsplit = max(1, min((keys + 63) // 64, 1024 // max(nblk, 1), 64))
            return _K.talking_attention_mfma(q, pool, int(heads), int(kv_heads), int(dim), int(vdim), float(scale),
                                             temp, talk, int(chunk), tiles, batch.cu_tokens, batch.start_pos,
                                             batch.block_tables, int(batch.block_size), int(nsplit))
        return _K.talking_attention(q, pool, int(heads), int(kv_heads), int(dim), int(vdim), float(scale), temp,
                                    talk, int(chunk), batch.tok_req, batch.tok_pos, batch.block_tables,
                                    int(batch.block_size))
    return ref.talking_attention(q, pool, heads, kv_heads, dim, vdim, scale, temp, talk, chunk, batch, out_dtype)


def gelu_tanh(z, out_dtype):
    if _native_k(z):
        return _K.gelu_tanh(z)
    return ref.gelu_tanh(z, out_dtype)


# ---------------------------------------------------------------------------
# ops of the gated extension: norms on both sides of a sublayer, restart of a
# repeated block of layers, rotation (pairs / halves) with unit norm and cache
# store, attention with one or two softmax maps a head, gated and differential
# finish, squared ReLU, experts without a gate matrix
# ---------------------------------------------------------------------------

scaled_freqs = ref.scaled_freqs
ROT_LAYOUTS = ref.ROT_LAYOUTS


def _native_g(x: torch.Tensor) -> bool:
    return _pick(x, "gated") is not None


def sandwich_norm_add(x, y, w_post, w_pre, eps, out_dtype, copy_to=None):
    """x fp32 [T, W] <- x + rms_unit(y) w_post in place (y may be None); ``copy_to`` (a [T, W]
    view of any row stride) receives the new x; -> rms_unit(x) w_pre in out_dtype, or None."""
    if _native_g(x):
        d = x.device
        h = _G.sandwich_norm_add(x, y if y is not None else _none(d), w_post if y is not None else _none(d),
                                 w_pre if w_pre is not None else _none(d), float(eps), out_dtype == torch.bfloat16,
                                 copy_to if copy_to is not None else _none(d))
        return h if w_pre is not None else None
    return ref.sandwich_norm_add(x, y, w_post, w_pre, eps, out_dtype, copy_to)


def restart_norm(y, bias, w_pre, eps, out_dtype):
    """-> (x fp32 = y + bias, rms_unit(x) w_pre in out_dtype)"""
    if _native_g(y):
        x, h = _G.restart_norm(y, bias, w_pre, float(eps), out_dtype == torch.bfloat16)
        return x, h
    return ref.restart_norm(y, bias, w_pre, eps, out_dtype)


def rope_norm_store(proj, q_heads, k_heads, dim, v_width, freqs, layout, unit_norm, eps, pool, batch):
    if _native_g(proj):
        return _G.rope_norm_store(proj, int(q_heads), int(k_heads), int(dim), int(v_width), freqs,
                                  ROT_LAYOUTS[layout], bool(unit_norm), float(eps), pool, batch.tok_pos,
                                  batch.tok_row)
    return ref.rope_norm_store(proj, q_heads, k_heads, dim, v_width, freqs, layout, unit_norm, eps, pool, batch)


def _map_mfma_ok(q, dim, vdim) -> bool:
    return (q.dtype == torch.bfloat16 and dim % 8 == 0 and vdim % 8 == 0 and dim <= 256 and vdim <= 256
            and os.environ.get("MEGATRON_AMD_NO_MFMA_MAPS", "0") != "1")


def _map_split(batch, nblk, vdim):
    """Key splits of the matrix-core kernel for steps with few row tiles.  Every split writes fp32
    partial results of vdim columns a row, so few long splits beat many short ones: measured best
    (4 and 16 requests at 2048 positions) at about 512 workgroups for values up to 128 wide and 256
    for wider ones (MEGATRON_AMD_MAP_SPLIT_WGS overrides)."""
    wgs = int(os.environ.get("MEGATRON_AMD_MAP_SPLIT_WGS", "512" if vdim <= 128 else "256"))
    return max(1, min((batch.max_context + 63) // 64, wgs // max(nblk, 1), 64))


def _map_tiles(batch, rep, key_heads, device):
    """Work list of the matrix-core kernel -> (tiles, rows a tile).  64 rows a workgroup (one row
    tile a wave); MEGATRON_AMD_MAP_TILE_ROWS=128 selects two row tiles a wave, which measured
    slower on whole prompts (more registers, fewer waves a SIMD) and is kept for experiments."""
    rows = int(os.environ.get("MEGATRON_AMD_MAP_TILE_ROWS", "64"))
    return batch.row_tiles(rep, device, rows), rows


def map_attention(q, pool, heads, kv_heads, maps, dim, vdim, scale, softcap, batch):
    """-> fp32 [T, heads * maps * vdim]: the result of every softmax map of every head"""
    if _native_g(q):
        if _map_mfma_ok(q, dim, vdim):
            tiles, rows = _map_tiles(batch, heads // kv_heads, kv_heads * maps, q.device)
            nsplit = _map_split(batch, tiles.shape[0] * kv_heads * maps, vdim)
            return _G.map_attention_mfma(q, _none(q.device), pool, int(heads), int(kv_heads), int(maps), int(dim),
                                         int(vdim), float(scale), float(softcap), tiles, batch.cu_tokens,
                                         batch.start_pos, batch.block_tables, int(batch.block_size), int(nsplit),
                                         rows)
        return _G.map_attention(q, pool, int(heads), int(kv_heads), int(maps), int(dim), int(vdim), float(scale),
                                float(softcap), batch.tok_req, batch.tok_pos, batch.block_tables,
                                int(batch.block_size))
    return ref.map_attention(q, pool, heads, kv_heads, maps, dim, vdim, scale, softcap, batch)


def softcap_gated_attention(q, gate, pool, heads, kv_heads, dim, vdim, scale, softcap, batch):
    """Causal grouped-query attention with capped scores whose concatenated heads
    are multiplied by sigmoid(gate [T, heads*vdim]) -> [T, heads*vdim] in q's dtype."""
    if _native_g(q):
        if _map_mfma_ok(q, dim, vdim):
            # matrix-core kernel, gate applied when the result leaves the accumulators
            tiles, rows = _map_tiles(batch, heads // kv_heads, kv_heads, q.device)
            nsplit = _map_split(batch, tiles.shape[0] * kv_heads, vdim)
            return _G.map_attention_mfma(q, gate, pool, int(heads), int(kv_heads), 1, int(dim), int(vdim),
                                         float(scale), float(softcap), tiles, batch.cu_tokens, batch.start_pos,
                                         batch.block_tables, int(batch.block_size), int(nsplit), rows)
        A = map_attention(q, pool, heads, kv_heads, 1, dim, vdim, scale, softcap, batch)
        return _G.gate_finish(A, gate, q.dtype == torch.bfloat16)
    A = ref.map_attention(q, pool, heads, kv_heads, 1, dim, vdim, scale, softcap, batch)
    return ref.gate_finish(A, gate, q.dtype)


def differential_attention(q, gate, lam, diff, eps, pool, heads, kv_heads, dim, vdim, scale, batch):
    """Two softmax maps a head over the same values: o = a1 - lam a2, unit-normed
    per head, times (1 - diff) sigmoid(gate [T, heads]) -> [T, heads*vdim] in q's dtype."""
    A = map_attention(q, pool, heads, kv_heads, 2, dim, vdim, scale, 0.0, batch)
    if _native_g(q):
        return _G.differential_finish(A, gate, lam, float(diff), float(eps), int(heads), int(vdim),
                                      q.dtype == torch.bfloat16)
    return ref.differential_finish(A, gate, lam, diff, eps, heads, vdim, q.dtype)


def relu2(z, out_dtype):
    if _native_g(z):
        return _G.relu2(z)
    return ref.relu2(z, out_dtype)


def expert_pairs_plain(h, ids, w_up, w_down):
    """Experts without a gate matrix, down(relu(up x)^2), one (token, choice) pair a row."""
    if _native_g(h):
        return _G.expert_pairs_plain(h, ids, w_up, w_down)
    return ref.expert_pairs_plain(h, ids, w_up, w_down)
