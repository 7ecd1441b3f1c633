"""Grouped-query softmax attention with rotated, unit-normed q and k, capped
scores and an elementwise sigmoid gate on the heads' outputs.

Per token, from one fused projection without bias [q | k | v | gate]:
  * the first ``rot_dims`` entries of every q and k head are rotated by the
    angle position * f_i, entry pairs (2i, 2i+1) (``layout="pairs"``) or
    (i, i + rot_dims/2) (``"halves"``); f_i = rot_base^(-2i/rot_dims), optionally
    rescaled by wavelength (ops.ragged.scaled_freqs); other entries pass,
  * ``unit_norm``: AFTER the rotation every q and k head is divided by its own
    root mean square (no weight),
  * score(i, j) = q(i) . k(j) * scale, then cap * tanh(score / cap) when a cap
    is given; position i sees every j <= i; softmax over the visible keys,
  * the concatenated heads (heads * vdim) are multiplied by
    sigmoid(gate projection of the same input), then the output projection.

Cache: one paged pool of a HybridInferenceContext under the name the caller
passes (a layer that runs several times a step keeps one pool per run), rows
[k | v] per token, k rotated and normed.  The step's own rows are written
before attention, so whole prompts, portions and decoded tokens are one path.
Angles, norms, scores, the cap, softmax and the gate are fp32."""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class GatedSoftcapAttention(nn.Module):
    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float,
                 softcap: Optional[float] = None, rot_dims: int = 0, rot_base: float = 10000.0,
                 rot_scaling: Optional[dict] = None, layout: str = "pairs", unit_norm: bool = True,
                 dtype=torch.bfloat16):
        super().__init__()
        assert heads % kv_heads == 0, "query heads are a multiple of key/value heads"
        assert rot_dims % 2 == 0 and 0 <= rot_dims <= dim, "rotated entries come in pairs inside a head"
        assert layout in R.ROT_LAYOUTS
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps = float(scale), float(eps)
        self.softcap = float(softcap) if softcap else 0.0
        self.layout, self.unit_norm = layout, bool(unit_norm)
        self.q_width, self.k_width, self.v_width = heads * dim, kv_heads * dim, kv_heads * vdim
        self.g_width = heads * vdim
        self.w_in = nn.Parameter(torch.zeros(self.q_width + self.k_width + self.v_width + self.g_width, hidden,
                                             dtype=dtype))                       # [q; k; v; gate]
        self.w_out = nn.Parameter(torch.zeros(hidden, heads * vdim, dtype=dtype))
        self.register_buffer("freqs", R.scaled_freqs(rot_dims, rot_base, rot_scaling), persistent=False)

    def cache_spec(self, name: str, page: int = 64):
        return {name: self.k_width + self.v_width}

    def forward(self, h: torch.Tensor, ctx, name: str) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        q = R.rope_norm_store(proj, self.heads, self.kv_heads, self.dim, self.v_width, self.freqs, self.layout,
                              self.unit_norm, self.eps, ctx.pools[name], ctx.batch)
        gate = proj[:, self.q_width + self.k_width + self.v_width:]
        o = R.softcap_gated_attention(q, gate, ctx.pools[name], self.heads, self.kv_heads, self.dim, self.vdim,
                                      self.scale, self.softcap, ctx.batch)
        return F.linear(o, self.w_out)
