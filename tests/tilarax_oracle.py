"""Plain per-sequence implementation of the Tilarax design, one function per
mechanism, for tests.  It shares no code with megatron_amd: whole sequences,
dense score matrices, python loops over tokens for the recurrence, float64 or
float32 torch tensors on the CPU.

A model is (config dict, {tensor name: tensor}); linear weights are [out, in].

Notation: T tokens, W width, H query heads, G key/value heads, d key size,
e value size, C chunk size, L layers.
"""

from __future__ import annotations

import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rotate_pairs(x, pos, dims, base):
    """x [T, heads, d]: the first ``dims`` entries of every head are rotated in
    neighbouring pairs (2i, 2i+1) by the angle pos * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    ang = pos.to(x.dtype).view(T, 1, 1) * freq.view(1, 1, half)
    c, s = torch.cos(ang), torch.sin(ang)
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def chunk_mask(T, size):
    """[T, T] bool: j <= i and both in the same run of ``size`` positions."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    return (j <= i) & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))


def talking_softmax_attention(q, k, v, scale, temp, talk, size):
    """q [T, H, d], k [T, G, d], v [T, G, e] of one whole sequence -> [T, H * e].
    Dense: every head's softmax over the visible keys, the weights mixed over
    the heads by ``talk``, head h then reads the values of its own key/value head."""
    T, H = q.shape[0], q.shape[1]
    rep = H // k.shape[1]
    mask = chunk_mask(T, size) if size else chunk_mask(T, T)
    probs = []
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd // rep].T) * scale * temp[hd]
        s = s.masked_fill(~mask, float("-inf"))
        probs.append(torch.softmax(s, dim=-1))
    mixed = torch.einsum("hg,gij->hij", talk, torch.stack(probs))
    return torch.cat([mixed[hd] @ v[:, hd // rep] for hd in range(H)], dim=-1)


def attention_mixer(h, m, w, p, eps, v_first):
    """h [T, W]; m the layer's mixer config; w tensors; p the tensor prefix.
    -> (output [T, W], the values this layer caches [T, G, e])"""
    T = h.shape[0]
    H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, d)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, d)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, e)
    q = rms(q, eps) * w[p + "q.norm"]
    k = rms(k, eps) * w[p + "k.norm"]
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot:
        q = rotate_pairs(q, pos, rot["dims"], rot["base"])
        k = rotate_pairs(k, pos, rot["dims"], rot["base"])
    if m.get("v_mix") and v_first is not None:
        lam = w[p + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    size = (m.get("mask") or {}).get("size")
    o = talking_softmax_attention(q, k, v, m["scale"], w[p + "temp"], w[p + "talk"], size)
    return o @ w[p + "o"].T + w[p + "o.b"], v


def mlstm_mixer(h, m, w, p, eps):
    T = h.shape[0]
    H, d, e, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[p + "k"].T).view(T, H, d)
    v = (h @ w[p + "v"].T).view(T, H, e)
    gi = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    out = torch.zeros(T, H, e, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(d, e, dtype=h.dtype)
        n = torch.zeros(d, dtype=h.dtype)
        mx = torch.zeros((), dtype=h.dtype)
        for t in range(T):
            new = torch.maximum(gf[t, hd] + mx, gi[t, hd])
            a, b = torch.exp(gf[t, hd] + mx - new), torch.exp(gi[t, hd] - new)
            S = a * S + b * torch.outer(k[t, hd], v[t, hd])
            n = a * n + b * k[t, hd]
            mx = new
            den = torch.maximum((n @ q[t, hd]).abs(), torch.exp(-mx)) + 1e-6
            out[t, hd] = (S.T @ q[t, hd]) / den
    o = rms(out, eps).reshape(T, H * e) * w[p + "norm"]
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def dense_ff(h, w, p):
    return gelu_tanh(h @ w[p + "up"].T) @ w[p + "down"].T


def route(h, r, w, p):
    """-> (ids [T, top], weights [T, top])"""
    z = h @ w[p + "router"].T + w[p + "router.b"]
    top, ids = torch.topk(z, r["top"], dim=-1)
    return ids, torch.softmax(top, dim=-1)


def moe_ff(h, mlp, w, p):
    ids, wt = route(h, mlp["router"], w, p)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(ids.shape[1]):
            q = f"{p}e{int(ids[t, c])}."
            y = silu(h[t] @ w[q + "gate"].T) * (h[t] @ w[q + "up"].T)
            out[t] += wt[t, c] * (y @ w[q + "down"].T)
    return out


def feed_forward(h, mlp, w, p):
    if mlp["kind"] == "dense":
        return dense_ff(h, w, p)
    return moe_ff(h, mlp, w, p)


def forward(cfg, w, tokens, dtype=torch.float64, layers_out=None):
    """tokens: list of ids -> logits [T, vocab]; ``layers_out`` (a list)
    receives what every layer hands on."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens)]
    hist = [x]
    v_first = None
    for i, lay in enumerate(cfg["layers"]):
        p = f"l{i}."
        if lay["type"] == "attention":
            y, v = attention_mixer(x, lay["mixer"], w, p + "mix.", eps, v_first)
            if lay["mixer"].get("v_mix") and v_first is None:
                v_first = v
        elif lay["type"] == "mlstm":
            y = mlstm_mixer(x, lay["mixer"], w, p + "mix.", eps)
        else:
            raise ValueError(lay["type"])
        x = x + norm_one_plus(y, w[p + "norm1"], eps)
        if lay.get("mlp"):
            x = x + norm_one_plus(feed_forward(x, lay["mlp"], w, p + "mlp."), w[p + "norm2"], eps)
        hist.append(x)
        x = sum(w[p + "dwa"][j] * hist[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x)
    x = norm_one_plus(x, w["final.norm"], eps)
    return x @ w["embed"].T
