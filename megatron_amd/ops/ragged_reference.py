"""Torch implementations of the ragged-batch sequence ops (CPU path).

Every op works on a flat batch of T tokens described by a
``RaggedBatch`` (megatron_amd/inference/contexts.py): request r brings tokens
``cu_tokens[r]:cu_tokens[r+1]`` at positions ``start_pos[r]...``; per-sequence
state lives in ``[num_slots, ...]`` tensors indexed by ``slots[r]`` and is
updated in place; paged caches are ``[rows, width]`` pools addressed through the
block tables.  The HIP kernels in csrc/ragged implement the same interfaces.

Precision rules (same as the kernels): norms, recurrences, gates, angles,
scores and softmax weights are computed in 32-bit whatever the tensors'
storage dtype; outputs are rounded once, on store.
"""

from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def _spans(batch):
    for r in range(batch.num_requests):
        yield r, batch.host_cu[r], batch.host_cu[r + 1], batch.host_start[r], batch.host_slots[r]


def embed_tokens(tokens, batch, embed, bigram, pos, prev_state, mul_prev, mul_cur, buckets):
    """x[t] = embed[tok] (+ bigram[hash(prev, tok)]) (+ pos[p]) in fp32.

    The hashed-bigram row is ``(prev * mul_prev + tok * mul_cur) % buckets``; a
    sequence's first token uses the extra row ``buckets``.  ``prev_state[slot]``
    carries the last token across steps."""
    x = embed[tokens].float()
    if bigram is not None:
        prev = torch.roll(tokens, 1)
        first_idx = batch.cu_tokens[:-1].long()
        prev[first_idx] = prev_state[batch.slots.long()].to(prev.dtype)
        row = (prev * mul_prev + tokens * mul_cur) % buckets
        row = torch.where(batch.tok_pos == 0, torch.full_like(row, buckets), row)
        x = x + bigram[row].float()
        last_idx = batch.cu_tokens[1:].long() - 1
        prev_state[batch.slots.long()] = tokens[last_idx].to(prev_state.dtype)
    if pos is not None:
        x = x + pos[batch.tok_pos.long()].float()
    return x


def hc_mix_norm(streams, y, mix, out_w, in_w, norm_w, eps):
    """Hyper-connection stream update fused with the next read and its norm.

    streams [T, S, W] fp32 (updated in place when ``y`` is given):
        x_t <- sum_s mix[s, t] x_s + out_w[t] * y
    then, when ``in_w`` is given, u = sum_s in_w[s] x_s and the result is
    ``u / sqrt(mean(u^2) + eps) * (1 + norm_w)`` in fp32 ([T, W])."""
    if y is not None:
        new = torch.einsum("st,nsw->ntw", mix.float(), streams) + out_w.float()[None, :, None] * y.float()[:, None, :]
        streams.copy_(new)
    if in_w is None:
        return None
    u = torch.einsum("s,nsw->nw", in_w.float(), streams)
    u = u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps)
    return u * (1.0 + norm_w.float())


def canon_conv(h, weight, state, batch, out_dtype):
    """h + causal depthwise conv over time of h, per request, with the last
    ``taps - 1`` inputs of earlier steps read from (and left in) ``state``
    [slots, taps-1, W].  weight [W, taps]: out_t = h_t + sum_j w[:, j] h_{t-taps+1+j}."""
    taps = weight.shape[1]
    out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
    wf = weight.float()
    for r, a, b, start, slot in _spans(batch):
        hist = torch.cat([state[slot], h[a:b].float()], dim=0)  # [taps-1 + n, W]
        n = b - a
        acc = h[a:b].float().clone()
        for j in range(taps):
            acc += wf[:, j] * hist[j : j + n]
        out[a:b] = acc.to(out_dtype)
        state[slot] = hist[n:]
    return out


def mingru_scan(zxg, bias_z, bias_x, state, batch, out_dtype):
    """minGRU over a ragged batch.  zxg [T, 3C]: pre-activations of the update
    gate, the candidate and the output gate.  z = sigmoid(. + bz); u = . + bx;
    cand = u + 1/2 (u >= 0) | sigmoid(u); S <- (1 - z) S + z cand; out = S * silu(g).
    state [slots, C] fp32."""
    C = zxg.shape[1] // 3
    z = torch.sigmoid(zxg[:, :C].float() + bias_z.float())
    u = zxg[:, C : 2 * C].float() + bias_x.float()
    g = zxg[:, 2 * C :].float()
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    out = torch.empty(zxg.shape[0], C, dtype=torch.float32, device=zxg.device)
    for r, a, b, start, slot in _spans(batch):
        S = state[slot].clone()
        for t in range(a, b):
            S = (1 - z[t]) * S + z[t] * cand[t]
            out[t] = S
        state[slot] = S
    return (out * F.silu(g)).to(out_dtype)


def mlstm_scan(qkvg, gates, bias_i, bias_f, norm_w, heads, dim, vdim, cap, eps,
               state_S, state_n, state_m, batch, out_dtype):
    """Stabilised matrix-memory recurrence (mLSTM) over a ragged batch.

    qkvg [T, H*dim | H*dim | H*vdim | H*vdim] (q unscaled, k, v, output-gate
    pre-activation); gates [T, 2H] fp32 pre-activations of the input and forget
    gates.  Log gates are soft-capped: i = cap tanh((. + bi)/cap),
    f = logsigmoid(cap tanh((. + bf)/cap)).  With running maximum m (0 at start):
        m' = max(f + m, i); S' = e^{f+m-m'} S + e^{i-m'} k v^T; n' likewise with k
        o = S'^T q / (max(|n'.q|, e^{-m'}) + 1e-6),  q scaled by dim^-1/2.
    Each head's o is RMS-normalised, scaled by norm_w and gated by sigmoid(g).
    States: S [slots, H, dim, vdim], n [slots, H, dim], m [slots, H], fp32."""
    T = qkvg.shape[0]
    H, D, V = heads, dim, vdim
    q, k, v, g = torch.split(qkvg.float(), [H * D, H * D, H * V, H * V], dim=1)
    q = q.view(T, H, D) * (D ** -0.5)
    k = k.view(T, H, D)
    v = v.view(T, H, V)
    ig = cap * torch.tanh((gates[:, :H].float() + bias_i.float()) / cap)
    fg = F.logsigmoid(cap * torch.tanh((gates[:, H:].float() + bias_f.float()) / cap))
    o = torch.empty(T, H, V, dtype=torch.float32, device=qkvg.device)
    for r, a, b, start, slot in _spans(batch):
        S, n, m = state_S[slot].clone(), state_n[slot].clone(), state_m[slot].clone()
        for t in range(a, b):
            m_new = torch.maximum(fg[t] + m, ig[t])
            da = torch.exp(fg[t] + m - m_new)
            db = torch.exp(ig[t] - m_new)
            S = da[:, None, None] * S + db[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
            n = da[:, None] * n + db[:, None] * k[t]
            m = m_new
            num = torch.einsum("hdv,hd->hv", S, q[t])
            den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            o[t] = num / den[:, None]
        state_S[slot], state_n[slot], state_m[slot] = S, n, m
    o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps)
    o = o.reshape(T, H * V) * norm_w.float() * torch.sigmoid(g)
    return o.to(out_dtype)


def rope_table(max_pos, dims, base, scaling=None, device=None):
    """cos/sin tables [max_pos, dims/2] fp32 for rotate-half RoPE with optional
    YaRN frequency interpolation.  scaling: dict(factor, original, fast, slow).
    Frequencies are blended between f_i and f_i / factor by a linear ramp over
    the pair index between the 'fast' and 'slow' rotation counts; cos and sin
    carry the YaRN magnitude factor 0.1 ln(factor) + 1."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    mag = 1.0
    if scaling:
        def pair_of(turns):
            return dims * math.log(scaling["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(pair_of(scaling["fast"])), 0)
        hi = min(math.ceil(pair_of(scaling["slow"])), dims - 1)
        ramp = ((torch.arange(half, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / scaling["factor"] * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(scaling["factor"]) + 1.0
    ang = torch.arange(max_pos, dtype=torch.float32)[:, None] * f.to(torch.float32)[None, :]
    return (torch.cos(ang) * mag).to(device), (torch.sin(ang) * mag).to(device)


def _rotate(x, cos, sin, dims):
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def latent_kv_store(dkv, norm_w, eps, cos, sin, rot_dims, rank, pool, batch):
    """Write each token's cache row: [RMS-normed latent * norm_w | rotated
    shared key part].  dkv [T, rank + rot_dim]; pool [rows, rank + rot_dim]."""
    c = dkv[:, :rank].float()
    c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * norm_w.float()
    p = batch.tok_pos.long()
    kr = _rotate(dkv[:, rank:].float(), cos[p], sin[p], rot_dims)
    pool[batch.tok_row] = torch.cat([c, kr], dim=-1).to(pool.dtype)


def latent_q_prepare(dq, norm_w, eps, out_dtype):
    """RMS norm with a plain weight over the query latent."""
    c = dq.float()
    return (c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * norm_w.float()).to(out_dtype)


def rope_heads(x, cos, sin, rot_dims, batch):
    """Rotate the first rot_dims dims of every head.  x [T, H, d]."""
    p = batch.tok_pos.long()
    return _rotate(x.float(), cos[p][:, None, :], sin[p][:, None, :], rot_dims).to(x.dtype)


def latent_sink_attention(q, pool, rank, sink, scale, batch):
    """Causal attention of absorbed queries over the paged latent cache.

    q [T, H, rank + rot] scores every cached row [latent | rotated key] of its
    own request up to its position; values are the rows' first ``rank`` entries
    (the value up-projection is applied by the caller).  The softmax
    denominator also holds exp(sink[h]): a per-head logit with no key or value."""
    T, H, Dk = q.shape
    out = torch.empty(T, H, rank, dtype=torch.float32, device=q.device)
    bs = batch.block_size
    for r, a, b, start, slot in _spans(batch):
        L = start + (b - a)
        table = torch.as_tensor(batch.host_tables[r], dtype=torch.long, device=q.device)
        rows = (table[:, None] * bs + torch.arange(bs, device=q.device)[None, :]).reshape(-1)[:L]
        kv = pool[rows].float()                               # [L, Dk]
        s = torch.einsum("thd,ld->thl", q[a:b].float(), kv) * scale
        qpos = torch.arange(start, L, device=q.device)
        mask = torch.arange(L, device=q.device)[None, :] > qpos[:, None]
        s = s.masked_fill(mask[:, None, :], float("-inf"))
        s = torch.cat([s, sink.float().view(1, H, 1).expand(b - a, H, 1)], dim=-1)
        p = torch.softmax(s, dim=-1)[..., :L]
        out[a:b] = torch.einsum("thl,lr->thr", p, kv[:, :rank])
    return out.to(q.dtype)


def xielu(z, act, out_dtype):
    """xIELU with raw parameters act = (p, q): for z > 0, softplus(p) z^2 + z/2;
    else (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    zf = z.float()
    ap = F.softplus(act[0].float())
    aq = 0.5 + F.softplus(act[1].float())
    pos = ap * zf * zf + 0.5 * zf
    neg = aq * (torch.expm1(torch.clamp(zf, max=0.0)) - zf) + 0.5 * zf
    return torch.where(zf > 0, pos, neg).to(out_dtype)


def gate_heads(x, gate_pre, heads):
    """x [T, H, d] (any strides) times sigmoid(gate_pre [T, H]) per head -> [T, H*d]."""
    T = x.shape[0]
    g = torch.sigmoid(gate_pre.float())
    return (x.float() * g[:, :, None]).reshape(T, -1).to(x.dtype)


# ---------------------------------------------------------------------------
# grouped RMS norm on a plain fp32 residual, attention over a sliding window
# plus mean-pooled blocks, generalized delta rule, routed clamped-GLU experts
# ---------------------------------------------------------------------------


def embed_plain(tokens, embed):
    """x[t] = embed[tok] in fp32."""
    return embed[tokens].float()


def residual_group_norm(x, y, w_a, w_b, groups, eps, out_dtype):
    """x [T, W] fp32 <- x + y (in place, when ``y`` is given), then RMS norm in
    ``groups`` equal consecutive parts (each divided by its own root mean square)
    times a plain weight; one normed copy per weight given (w_b may be None)."""
    if y is not None:
        x.add_(y.float())
    T, W = x.shape
    p = x.view(T, groups, W // groups)
    n = (p * torch.rsqrt((p * p).mean(-1, keepdim=True) + eps)).reshape(T, W)
    h_a = (n * w_a.float()).to(out_dtype)
    h_b = (n * w_b.float()).to(out_dtype) if w_b is not None else None
    return h_a, h_b


def qk_norm_store(proj, q_off, q_width, k_off, k_width, v_off, v_width, q_norm, k_norm, eps, pool, batch):
    """From the fused projection rows ``proj`` [T, *]: RMS norm of the whole query
    slice (all heads at once) and of the whole key slice with plain weights;
    the cache row of each token becomes [normed keys | values], the values
    being the slice at ``v_off`` as projected.  Returns the normed queries."""
    def norm(z, w):
        z = z.float()
        return z * torch.rsqrt((z * z).mean(-1, keepdim=True) + eps) * w.float()
    q = norm(proj[:, q_off:q_off + q_width], q_norm).to(proj.dtype)
    k = norm(proj[:, k_off:k_off + k_width], k_norm)
    pool[batch.tok_row] = torch.cat([k, proj[:, v_off:v_off + v_width].float()], dim=-1).to(pool.dtype)
    return q


def _rows_of(table, n, per_page, device):
    """cache rows of a request's entries 0..n-1 in a pool with per_page rows a page"""
    idx = torch.arange(n, device=device)
    return table[idx // per_page] * per_page + idx % per_page


def pool_blocks(pool, pooled, block, pooled_per_page, batch):
    """Mean of every block of ``block`` consecutive cache rows that this step
    completed (its last position was written now), as the cache holds them,
    into the pooled pool (entry b of a request = block b)."""
    bs = batch.block_size
    for r, a, b, start, slot in _spans(batch):
        first, last = start // block, (start + b - a) // block
        if last <= first:
            continue
        table = torch.as_tensor(batch.host_tables[r], dtype=torch.long, device=pool.device)
        rows = _rows_of(table, last * block, bs, pool.device)[first * block:]
        mean = pool[rows].float().view(last - first, block, -1).mean(1)
        prow = _rows_of(table, last, pooled_per_page, pool.device)[first:]
        pooled[prow] = mean.to(pooled.dtype)


def pooled_window_attention(q, pool, pooled, heads, kv_heads, dim, vdim, scale, window, block,
                            pooled_per_page, batch, out, out_col, out_scale):
    """Grouped-query softmax attention over the paged cache where position i sees
    the tokens j with 0 <= i - j < window and, beside them, one mean-pooled
    key/value for each block of ``block`` tokens that ends at or before
    i - window.  Cache rows are [kv_heads * dim keys | kv_heads * vdim values].
    Writes out[:, out_col : out_col + heads * vdim] = out_scale * result."""
    T = q.shape[0]
    H, G, D, V = heads, kv_heads, dim, vdim
    rep = H // G
    bs = batch.block_size
    dev = q.device
    for r, a, b, start, slot in _spans(batch):
        n = b - a
        L = start + n
        table = torch.as_tensor(batch.host_tables[r], dtype=torch.long, device=dev)
        kv = pool[_rows_of(table, L, bs, dev)].float()
        nb_max = max(0, L - window) // block
        if nb_max > 0:
            pk = pooled[_rows_of(table, nb_max, pooled_per_page, dev)].float()
            kv = torch.cat([pk, kv], dim=0)
        keys = kv[:, :G * D].view(-1, G, D)
        vals = kv[:, G * D:].view(-1, G, V)
        qi = torch.arange(start, L, device=dev)
        j = torch.arange(L, device=dev)
        tok_ok = (j[None, :] <= qi[:, None]) & (qi[:, None] - j[None, :] < window)
        nb = torch.clamp(qi - window + 1, min=0) // block
        blk_ok = torch.arange(nb_max, device=dev)[None, :] < nb[:, None]
        ok = torch.cat([blk_ok, tok_ok], dim=1)                       # [n, nb_max + L]
        qq = q[a:b].float().view(n, G, rep, D)
        s = torch.einsum("ngrd,lgd->ngrl", qq, keys) * scale
        s = s.masked_fill(~ok[:, None, None, :], float("-inf"))
        p = torch.softmax(s, dim=-1)
        o = torch.einsum("ngrl,lgv->ngrv", p, vals).reshape(n, H * V)
        out[a:b, out_col:out_col + H * V] = (o * out_scale).to(out.dtype)


def delta_rule_scan(proj, r_off, k_off, v_off, g_off, a_off, w_off, w_rank, w2, w0, a_bias, norm_w,
                    heads, dim, eps, state, batch, out, out_col, out_scale):
    """Generalized delta rule over a ragged batch.  ``proj`` [T, *] holds, at the
    given column offsets, r, k, v, the output-gate and removal-rate
    pre-activations (heads * dim each) and the decay bottleneck (w_rank).
        decay   w = exp(-e^{-1/2} sigmoid(w2 tanh(.) + w0)),   removal a = sigmoid(. + a_bias)
        unit key u = k / sqrt(sum k^2 + 1e-6)  (per head)
        S <- diag(w) S - (a u)(u^T S) + k v^T  (both terms read the old S),  o = S^T r
    Each head's o is divided by its root mean square, times norm_w, times
    sigmoid(gate).  state [slots, heads, dim, dim] fp32.  Writes
    out[:, out_col : out_col + heads * dim] = out_scale * result."""
    T = proj.shape[0]
    H, D = heads, dim
    HD = H * D
    pf = proj.float()
    rr = pf[:, r_off:r_off + HD].view(T, H, D)
    k = pf[:, k_off:k_off + HD].view(T, H, D)
    v = pf[:, v_off:v_off + HD].view(T, H, D)
    g = pf[:, g_off:g_off + HD]
    z = torch.tanh(pf[:, w_off:w_off + w_rank]) @ w2.float().T + w0.float()
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(z)).view(T, H, D)
    al = torch.sigmoid(pf[:, a_off:a_off + HD] + a_bias.float()).view(T, H, D)
    u = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    o = torch.empty(T, H, D, dtype=torch.float32, device=proj.device)
    for r, a, b, start, slot in _spans(batch):
        S = state[slot].clone()
        for t in range(a, b):
            uS = torch.einsum("hd,hde->he", u[t], S)
            S = w[t][:, :, None] * S - (al[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hde,hd->he", S, rr[t])
        state[slot] = S
    o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps)
    o = o.reshape(T, HD) * norm_w.float() * torch.sigmoid(g)
    out[:, out_col:out_col + HD] = (o * out_scale).to(out.dtype)


def moe_route(logits, experts, top, groups, keep, scale):
    """Sigmoid scores of the first ``experts`` logit columns; the ``top`` largest
    are chosen, among the experts of the best ``keep`` of ``groups`` neighbour
    groups when groups > 1 (a group's score: sum of its two largest scores);
    weights = chosen scores / (their sum + 1e-20) * scale.
    -> (ids [T, top] int32, weights [T, top] fp32)."""
    from megatron_amd.moe.router import group_limited_topk

    s = torch.sigmoid(logits[:, :experts].float())
    if groups > 1:
        _, idx = group_limited_topk(s, top, groups, keep)
    else:
        idx = s.topk(top, dim=-1).indices
    sc = s.gather(1, idx)
    return idx.to(torch.int32), sc / (sc.sum(-1, keepdim=True) + 1e-20) * scale


def clamped_glu(gu, limit, alpha, out_dtype):
    """gu [N, 2F] = [gate | up]: g = min(gate, limit), u = clamp(up, -limit, limit),
    y = g sigmoid(alpha g) (u + 1)."""
    F_ = gu.shape[1] // 2
    g = torch.clamp(gu[:, :F_].float(), max=limit)
    u = torch.clamp(gu[:, F_:].float(), -limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(out_dtype)


def moe_combine(down, inv, weights, shared, shared_gate, add):
    """y[t] = sum_k weights[t, k] down[inv[t, k]] (+ sigmoid(shared_gate[t]) shared[t]) (+ add[t]), fp32."""
    T, K = weights.shape
    y = (down.float()[inv.long().view(-1)].view(T, K, -1) * weights[:, :, None]).sum(1)
    if shared is not None:
        y = y + torch.sigmoid(shared_gate.float())[:, None] * shared.float()
    if add is not None:
        y = y + add.float()
    return y


def expert_pairs(h, ids, w_gate_up, w_down, limit, alpha, act="clamped"):
    """Every (token, choice) pair through its expert, rows in pair order
    (token-major): GLU of [gate; up] x (clamped or SiLU), then the down product."""
    T, K = ids.shape
    out = torch.empty(T * K, h.shape[1], dtype=h.dtype, device=h.device)
    for t in range(T):
        for k in range(K):
            e = int(ids[t, k])
            gu = F.linear(h[t:t + 1], w_gate_up[e])
            y = silu_glu(gu, h.dtype) if act == "silu" else clamped_glu(gu, limit, alpha, h.dtype)
            out[t * K + k] = F.linear(y, w_down[e])[0]
    return out


def moe_router(h, w_router, experts, top, groups, keep, scale, bias=None, score="sigmoid"):
    """Router in one call: fp32 logits of all rows of w_router (+ bias; the rows
    beyond ``experts`` are returned raw), then moe_route (score "sigmoid") or
    moe_route_softmax (score "softmax") or moe_route_softmax_all (score
    "softmax_all").  -> (ids, weights, extra [T, rows - experts])"""
    logits = F.linear(h.float(), w_router.float(), bias.float() if bias is not None else None)
    if score == "softmax":
        ids, weights = moe_route_softmax(logits[:, :experts], top)
    elif score == "softmax_all":
        ids, weights = moe_route_softmax_all(logits[:, :experts], top)
    else:
        ids, weights = moe_route(logits, experts, top, groups, keep, scale)
    return ids, weights, logits[:, experts:].contiguous()


# ---------------------------------------------------------------------------
# post-sublayer norm with depth-weighted residual history, per-head q/k norm
# with pairwise rotation and value mixing, chunked talking-heads attention,
# tanh-GELU, routing by softmax over the chosen logits, SiLU GLU
# ---------------------------------------------------------------------------


def post_norm_add(x, y, w, eps, out_dtype, hist, depth, dwa):
    """x fp32 [T, W] <- x + y / sqrt(mean(y^2) + eps) * (1 + w) in place (skipped
    when ``y`` is None).  With ``hist`` ([layers + 1, T, W] fp32, entry 0 = the
    embedding output): hist[depth] <- x, then x <- sum_{j <= depth} dwa[j] hist[j].
    Returns x in ``out_dtype`` (the next sublayer's GEMM input)."""
    if y is not None:
        yf = y.float()
        x.add_(yf * torch.rsqrt((yf * yf).mean(-1, keepdim=True) + eps) * (1.0 + w.float()))
    if hist is not None:
        hist[depth].copy_(x)
        x.copy_(torch.einsum("j,jtw->tw", dwa.float()[:depth + 1], hist[:depth + 1]))
    return x if out_dtype == torch.float32 else x.to(out_dtype)


def pair_freqs(dims, base, device=None):
    """f_i = base^(-2i/dims), i < dims/2, rounded once to fp32."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims).to(torch.float32).to(device)


def _rotate_pairs(x, pos, freqs):
    """x [T, heads, d] fp32: entries (2i, 2i+1), i < len(freqs), rotated by pos * f_i."""
    n = freqs.numel()
    if n == 0:
        return x
    ang = pos.float()[:, None, None] * freqs.float()[None, None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out = x.clone()
    out[..., 0:2 * n:2] = u * c - v * s
    out[..., 1:2 * n:2] = v * c + u * s
    return out


def head_norm_rope_store(proj, heads, kv_heads, dim, vdim, q_norm, k_norm, eps, freqs, v_first, lam, pool, batch):
    """proj [T, H*dim | G*dim | G*vdim] = [q | k | v] of the step's tokens.
    Every head of q and k is divided by its own root mean square and scaled by a
    weight [dim] that all heads share, then its first 2 * len(freqs) entries are
    rotated in neighbouring pairs by the token's position.  With ``v_first``
    ([T, G*vdim], another layer's values of the same tokens):
    v <- (1 - lam) v + lam v_first.  Cache row <- [k | v]; returns q [T, H*dim]."""
    T = proj.shape[0]
    H, G, D, V = heads, kv_heads, dim, vdim
    pf = proj.float()
    q = pf[:, :H * D].view(T, H, D)
    k = pf[:, H * D:(H + G) * D].view(T, G, D)
    v = pf[:, (H + G) * D:(H + G) * D + G * V]
    q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_norm.float()
    k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_norm.float()
    q = _rotate_pairs(q, batch.tok_pos, freqs)
    k = _rotate_pairs(k, batch.tok_pos, freqs)
    if v_first is not None:
        lf = lam.float().reshape(())
        v = (1.0 - lf) * v + lf * v_first.float()
    pool[batch.tok_row] = torch.cat([k.reshape(T, G * D), v], dim=-1).to(pool.dtype)
    return q.reshape(T, H * D).to(proj.dtype)


def talking_attention(q, pool, heads, kv_heads, dim, vdim, scale, temp, talk, chunk, batch, out_dtype):
    """Softmax attention over the paged cache (rows [G*dim keys | G*vdim values])
    whose weights are mixed over the heads after the softmax:
        s_g(i, j) = q_g(i) . k_kv(g)(j) * scale * temp[g],   P_g = softmax_j s_g
        o_h(i) = sum_j (sum_g talk[h, g] P_g(i, j)) v_kv(h)(j)
    Position i sees j <= i with floor(j / chunk) = floor(i / chunk) (chunk <= 0:
    every j <= i).  -> [T, H*vdim]."""
    T = q.shape[0]
    H, G, D, V = heads, kv_heads, dim, vdim
    rep = H // G
    bs = batch.block_size
    dev = q.device
    out = torch.empty(T, H * V, dtype=out_dtype, device=dev)
    kvh = torch.arange(H, device=dev) // rep
    for r, a, b, start, slot in _spans(batch):
        n = b - a
        L = start + n
        lo = (start // chunk) * chunk if chunk > 0 else 0          # nothing older is visible to this step
        table = torch.as_tensor(batch.host_tables[r], dtype=torch.long, device=dev)
        kv = pool[_rows_of(table, L, bs, dev)[lo:]].float()
        keys = kv[:, :G * D].view(-1, G, D)
        vals = kv[:, G * D:].view(-1, G, V)
        qi = torch.arange(start, L, device=dev)
        j = torch.arange(lo, L, device=dev)
        ok = j[None, :] <= qi[:, None]
        if chunk > 0:
            ok = ok & (torch.div(j, chunk, rounding_mode="floor")[None, :]
                       == torch.div(qi, chunk, rounding_mode="floor")[:, None])
        qq = q[a:b].float().view(n, H, D)
        s = torch.einsum("nhd,lhd->nhl", qq, keys[:, kvh]) * (scale * temp.float())[None, :, None]
        s = s.masked_fill(~ok[:, None, :], float("-inf"))
        p = torch.softmax(s, dim=-1)
        pm = torch.einsum("hg,ngl->nhl", talk.float(), p)
        o = torch.einsum("nhl,lhv->nhv", pm, vals[:, kvh])
        out[a:b] = o.reshape(n, H * V).to(out_dtype)
    return out


def gelu_tanh(z, out_dtype):
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))"""
    zf = z.float()
    return (0.5 * zf * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (zf + 0.044715 * zf * zf * zf)))).to(out_dtype)


def silu_glu(gu, out_dtype):
    """gu [N, 2F] = [gate | up]: y = gate sigmoid(gate) up."""
    F_ = gu.shape[1] // 2
    g, u = gu[:, :F_].float(), gu[:, F_:].float()
    return (g * torch.sigmoid(g) * u).to(out_dtype)


def moe_route_softmax(logits, top):
    """The ``top`` largest logits are chosen; weights = softmax over the chosen
    logits only.  -> (ids [T, top] int32, weights [T, top] fp32)."""
    val, idx = logits.float().topk(top, dim=-1)
    return idx.to(torch.int32), torch.softmax(val, dim=-1)


# ---------------------------------------------------------------------------
# norms on both sides of a sublayer, restart of a repeated block of layers,
# rotation in pairs or halves with wavelength-dependent frequency scaling and an
# optional unit norm, attention with several softmax maps per head over shared
# values (capped scores, gated or differential finish), squared ReLU, routing by
# the softmax over all experts, experts without a gate matrix
# ---------------------------------------------------------------------------


def sandwich_norm_add(x, y, w_post, w_pre, eps, out_dtype, copy_to=None):
    """x fp32 [T, W] <- x + y / sqrt(mean(y^2) + eps) * w_post in place (skipped
    when ``y`` is None).  ``copy_to`` ([T, W] view, any row stride) receives the
    new x in its own dtype.  Returns x / sqrt(mean(x^2) + eps) * w_pre in
    ``out_dtype`` (None when ``w_pre`` is None)."""
    if y is not None:
        yf = y.float()
        x.add_(yf * torch.rsqrt((yf * yf).mean(-1, keepdim=True) + eps) * w_post.float())
    if copy_to is not None:
        copy_to.copy_(x)
    if w_pre is None:
        return None
    return (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w_pre.float()).to(out_dtype)


def restart_norm(y, bias, w_pre, eps, out_dtype):
    """A fresh fp32 residual x = y + bias (bias [W]) and its normed copy
    x / sqrt(mean(x^2) + eps) * w_pre in ``out_dtype``.  -> (x, h)"""
    x = y.float() + bias.float()
    return x, (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w_pre.float()).to(out_dtype)


def scaled_freqs(dims, base, scaling=None, device=None):
    """f_i = base^(-2i/dims), i < dims/2, in float64; with ``scaling`` (factor,
    low, high, original): a wavelength 2 pi / f below original/high keeps f, one
    above original/low uses f / factor, and between them
    s = (original / wavelength - low) / (high - low) blends (1 - s) f / factor + s f.
    Kept in float64: at position p the angle p f_i is formed in float64 and reduced to
    (-pi, pi] before it is rounded to fp32, so far positions lose no precision."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    if scaling:
        factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
        orig = float(scaling["original"])
        wl = 2.0 * math.pi / f
        s = (orig / wl - low) / (high - low)
        mid = (1.0 - s) * f / factor + s * f
        f = torch.where(wl < orig / high, f, torch.where(wl > orig / low, f / factor, mid))
    return f.to(device)


ROT_LAYOUTS = {"pairs": 0, "halves": 1}


def _rotate_layout(x, pos, freqs, layout):
    """x [T, heads, d] fp32; "pairs": entries (2i, 2i+1), "halves": (i, i + n),
    i < n = len(freqs), rotated by pos * f_i."""
    n = freqs.numel()
    if n == 0:
        return x
    ang = torch.remainder(pos.double()[:, None, None] * freqs.double()[None, None, :] + math.pi, 2.0 * math.pi) - math.pi
    ang = ang.float()
    c, s = torch.cos(ang), torch.sin(ang)
    out = x.clone()
    if layout == "pairs":
        u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = u * c - v * s
        out[..., 1:2 * n:2] = v * c + u * s
    else:
        u, v = x[..., :n], x[..., n:2 * n]
        out[..., :n] = u * c - v * s
        out[..., n:2 * n] = v * c + u * s
    return out


def rope_norm_store(proj, q_heads, k_heads, dim, v_width, freqs, layout, unit_norm, eps, pool, batch):
    """proj [T, q_heads*dim | k_heads*dim | v_width | ...] (columns beyond the
    values are not read).  Every q and k head is rotated by the token's position
    (``layout``: "pairs" or "halves", first 2 len(freqs) entries) and then, with
    ``unit_norm``, divided by its root mean square.  Cache row <- [k | v];
    returns q [T, q_heads*dim]."""
    T = proj.shape[0]
    D = dim
    pf = proj.float()
    q = pf[:, :q_heads * D].view(T, q_heads, D)
    k = pf[:, q_heads * D:(q_heads + k_heads) * D].view(T, k_heads, D)
    v = pf[:, (q_heads + k_heads) * D:(q_heads + k_heads) * D + v_width]
    q = _rotate_layout(q, batch.tok_pos, freqs, layout)
    k = _rotate_layout(k, batch.tok_pos, freqs, layout)
    if unit_norm:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps)
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps)
    pool[batch.tok_row] = torch.cat([k.reshape(T, k_heads * D), v], dim=-1).to(pool.dtype)
    return q.reshape(T, q_heads * D).to(proj.dtype)


def map_attention(q, pool, heads, kv_heads, maps, dim, vdim, scale, softcap, batch):
    """Causal softmax attention over the paged cache with ``maps`` softmax maps a
    head.  q [T, heads*maps*dim], head-major then map; cache rows
    [kv_heads*maps*dim keys | kv_heads*vdim values]: map m of query head h reads
    key (h // rep, m) and the values of key/value head h // rep.
        s = q . k * scale;  softcap > 0: s <- softcap tanh(s / softcap)
    -> fp32 [T, heads*maps*vdim]."""
    T = q.shape[0]
    H, G, M, D, V = heads, kv_heads, maps, dim, vdim
    rep = H // G
    bs = batch.block_size
    dev = q.device
    out = torch.empty(T, H * M * V, dtype=torch.float32, device=dev)
    hm = torch.arange(H * M, device=dev)
    key_of = (hm // (rep * M)) * M + hm % M
    val_of = hm // (rep * M)
    for r, a, b, start, slot in _spans(batch):
        n = b - a
        L = start + n
        table = torch.as_tensor(batch.host_tables[r], dtype=torch.long, device=dev)
        kv = pool[_rows_of(table, L, bs, dev)].float()
        keys = kv[:, :G * M * D].view(-1, G * M, D)
        vals = kv[:, G * M * D:].view(-1, G, V)
        qi = torch.arange(start, L, device=dev)
        j = torch.arange(L, device=dev)
        ok = j[None, :] <= qi[:, None]
        qq = q[a:b].float().view(n, H * M, D)
        s = torch.einsum("nhd,lhd->nhl", qq, keys[:, key_of]) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~ok[:, None, :], float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[a:b] = torch.einsum("nhl,lhv->nhv", p, vals[:, val_of]).reshape(n, H * M * V)
    return out


def gate_finish(A, gate, out_dtype):
    """A fp32 [T, N] * sigmoid(gate [T, N]) -> out_dtype"""
    return (A * torch.sigmoid(gate.float())).to(out_dtype)


def differential_finish(A, gate, lam, diff, eps, heads, vdim, out_dtype):
    """A fp32 [T, heads*2*vdim] = the two maps' results (a1, a2) per head;
    o = a1 - lam a2, o <- o / sqrt(mean(o^2) + eps) * (1 - diff), times
    sigmoid(gate[t, head]).  -> [T, heads*vdim] in out_dtype."""
    T = A.shape[0]
    a = A.view(T, heads, 2, vdim)
    o = a[:, :, 0] - lam.float().reshape(()) * a[:, :, 1]
    o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * (1.0 - diff)
    o = o * torch.sigmoid(gate.float())[:, :, None]
    return o.reshape(T, heads * vdim).to(out_dtype)


def relu2(z, out_dtype):
    """max(z, 0)^2"""
    r = torch.relu(z.float())
    return (r * r).to(out_dtype)


def gelu_glu(gu, out_dtype):
    """gu [N, 2F] = [gate | up]: y = gelu_tanh(gate) up."""
    F_ = gu.shape[1] // 2
    return (gelu_tanh(gu[:, :F_], torch.float32) * gu[:, F_:].float()).to(out_dtype)


def moe_route_softmax_all(logits, top):
    """Scores = softmax over ALL experts; the ``top`` largest are chosen and
    keep their own scores as weights (they do not sum to one).
    -> (ids [T, top] int32, weights [T, top] fp32)."""
    val, idx = torch.softmax(logits.float(), dim=-1).topk(top, dim=-1)
    return idx.to(torch.int32), val


def expert_pairs_plain(h, ids, w_up, w_down):
    """Every (token, choice) pair through its expert without a gate matrix,
    down(relu(up x)^2); rows in pair order (token-major)."""
    T, K = ids.shape
    out = torch.empty(T * K, h.shape[1], dtype=h.dtype, device=h.device)
    for t in range(T):
        for k in range(K):
            e = int(ids[t, k])
            out[t * K + k] = F.linear(relu2(F.linear(h[t:t + 1], w_up[e]), h.dtype), w_down[e])[0]
    return out
