"""A plain, slow implementation of the Lomazen design in float64, one function
per mechanism, one sequence at a time, no cache.  It shares no code with the
product path; tests compare the framework against it.

Notation: W width, H query heads, G key/value heads, D key size, V value size,
R rotated entries per head (or per map), T tokens of the sequence.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_unit(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotation_freqs(rot: Optional[dict]) -> List[float]:
    """f_i = base^(-2i/R), i < R/2, with the optional wavelength-dependent scaling:
    wavelengths under original/high keep f, above original/low use f/factor, and
    between them the two are blended linearly in original/wavelength."""
    if not rot or not rot.get("dims"):
        return []
    R, base = int(rot["dims"]), float(rot["base"])
    fs = [base ** (-2.0 * i / R) for i in range(R // 2)]
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for f in fs:
            wl = 2.0 * math.pi / f
            if wl < orig / high:
                out.append(f)
            elif wl > orig / low:
                out.append(f / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * f / factor + s * f)
        fs = out
    return fs


def rotate(x: torch.Tensor, freqs: List[float], layout: str) -> torch.Tensor:
    """x [T, n, D]; position = row index.  layout "pairs": entry 2i goes with
    2i+1; "halves": entry i goes with i + R/2.  Entries from R on pass."""
    n = len(freqs)
    if n == 0:
        return x
    T = x.shape[0]
    ang = torch.arange(T, dtype=F64)[:, None] * torch.tensor(freqs, dtype=F64)[None, :]   # [T, n]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if layout == "pairs":
        a, b = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = a * c - b * s
        out[..., 1:2 * n:2] = b * c + a * s
    else:
        a, b = x[..., :n], x[..., n:2 * n]
        out[..., :n] = a * c - b * s
        out[..., n:2 * n] = b * c + a * s
    return out


def causal_softmax(scores: torch.Tensor) -> torch.Tensor:
    """scores [T, T] (query, key) -> weights; query i sees keys j <= i."""
    T = scores.shape[0]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    return torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1)


def gated_attention(h: torch.Tensor, p: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Grouped-query attention with rotated then unit-normed q and k, capped
    scores and an elementwise sigmoid gate on the heads' outputs."""
    H, G, D, V = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, D)
    k = (h @ p["k"].T).view(T, G, D)
    v = (h @ p["v"].T).view(T, G, V)
    fr = rotation_freqs(m.get("rot"))
    q, k = rms_unit(rotate(q, fr, "pairs"), eps), rms_unit(rotate(k, fr, "pairs"), eps)
    cap = m.get("softcap")
    outs = []
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(m["scale"])
        if cap:
            s = float(cap) * torch.tanh(s / float(cap))
        outs.append(causal_softmax(s) @ v[:, g])
    o = torch.cat(outs, dim=-1)                                   # [T, H*V]
    o = o * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T


def differential_attention(h: torch.Tensor, p: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Two softmax maps per head over the same values, combined as
    a1 - lam a2, unit-normed per head, scaled by 1 - diff, one gate per head."""
    H, G, D, V = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    diff = float(m["diff"])
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H * 2, D)
    k = (h @ p["k"].T).view(T, G * 2, D)
    v = (h @ p["v"].T).view(T, G, V)
    fr = rotation_freqs(m.get("rot"))
    q, k = rotate(q, fr, "halves"), rotate(k, fr, "halves")
    lam = math.exp(float((p["lq1"] * p["lk1"]).sum())) - math.exp(float((p["lq2"] * p["lk2"]).sum())) + diff
    gate = torch.sigmoid(h @ p["g"].T)                            # [T, H]
    outs = []
    for hd in range(H):
        g = hd // (H // G)
        a = []
        for mp in range(2):
            s = (q[:, 2 * hd + mp] @ k[:, 2 * g + mp].T) * float(m["scale"])
            a.append(causal_softmax(s) @ v[:, g])
        o = rms_unit(a[0] - lam * a[1], eps) * (1.0 - diff)
        outs.append(o * gate[:, hd:hd + 1])
    return torch.cat(outs, dim=-1) @ p["o"].T


def dense_ff(h, p):
    return (gelu_tanh(h @ p["gate"].T) * (h @ p["up"].T)) @ p["down"].T


def routed_ff(h: torch.Tensor, p: Dict[str, torch.Tensor], spec: dict) -> torch.Tensor:
    """Softmax over all experts; the `top` largest are used with their own
    scores as weights (no renormalisation); expert = down(relu(up h)^2)."""
    E, top = int(spec["router"]["experts"]), int(spec["router"]["top"])
    s = torch.softmax(h @ p["router"].T, dim=-1)
    w, ids = torch.topk(s, top, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            y = torch.relu(h[t] @ p[f"e{e}.up"].T) ** 2
            out[t] += w[t, j] * (y @ p[f"e{e}.down"].T)
    return out


def sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(F64) for k, v in tensors.items() if k.startswith(prefix)}


def layer(x, i, spec, tensors, eps):
    p = sub(tensors, f"l{i}.")
    mix = {"attention": gated_attention, "attention_2": differential_attention}[spec["type"]]
    x = x + rms_norm(mix(rms_norm(x, p["norm1"], eps), sub(tensors, f"l{i}.mix."), spec["mixer"], eps),
                     p["norm1b"], eps)
    mlp = spec.get("mlp")
    if mlp:
        q = sub(tensors, f"l{i}.mlp.")
        hh = rms_norm(x, p["norm2"], eps)
        y = dense_ff(hh, q) if mlp.get("kind", "dense") == "dense" else routed_ff(hh, q, mlp)
        x = x + rms_norm(y, p["norm2b"], eps)
    return x


def schedule(cfg: dict):
    """(layer index, pass number, first of its pass) for every layer run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, 0, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, 0, False) for i in range(a)]
    for t in range(times):
        runs += [(i, t, i == a) for i in range(a, b)]
    runs += [(i, 0, False) for i in range(b, n)]
    return runs


def model(tokens: List[int], cfg: dict, tensors: Dict[str, torch.Tensor], trace: Optional[list] = None):
    """-> logits [T, vocab] float64"""
    eps = float(cfg["norm"]["eps"])
    emb = tensors["embed"].to(F64)
    x0 = emb[torch.tensor(tokens)]
    x = x0
    for i, t, first in schedule(cfg):
        if first:
            x = torch.cat([x, x0], dim=-1) @ tensors["loop.in"].to(F64).T + tensors["loop.step"].to(F64)[t]
        x = layer(x, i, cfg["layers"][i], tensors, eps)
        if trace is not None:
            trace.append(x.clone())
    x = rms_norm(x, tensors["final.norm"].to(F64), eps)
    return (x @ emb.T) * float(cfg.get("logit_scale", 1.0))
