"""Differential grouped-query attention: every head holds TWO softmax maps over
the same values and outputs their weighted difference.

Per token, from one fused projection without bias [q | k | v | gate]; q has
heads * 2 * dim entries and k has kv_heads * 2 * dim, head by head as
[map 1 | map 2]:
  * the first ``rot_dims`` entries of every map of every q and k head are
    rotated by position * f_i (``layout="halves"``: entry i with i + rot_dims/2;
    ``"pairs"``: 2i with 2i+1), f_i = rot_base^(-2i/rot_dims),
  * each map is a causal softmax attention of its own,
    s_m(i, j) = q_m(i) . k_m(j) * scale, a_m = softmax(s_m) v,
  * lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number for the layer,
    o = a_1 - lam a_2, divided by its root mean square over the head's values
    (no weight) and multiplied by (1 - diff),
  * head h's result is multiplied by sigmoid(gate_h), ONE gate per head from
    the same input as the projections; then the output projection.

Cache: one paged pool under the caller's name, rows [k (both maps) | v].
Angles, scores, softmax, a_m, lam, the difference, its norm and the gate are
fp32 (ops.ragged.differential_attention)."""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class DifferentialAttention(nn.Module):
    maps = 2

    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float,
                 diff: float, rot_dims: int = 0, rot_base: float = 10000.0, rot_scaling: Optional[dict] = None,
                 layout: str = "halves", dtype=torch.bfloat16):
        super().__init__()
        assert heads % kv_heads == 0, "query heads are a multiple of key/value heads"
        assert rot_dims % 2 == 0 and 0 <= rot_dims <= dim, "rotated entries come in pairs inside a map"
        assert layout in R.ROT_LAYOUTS
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps, self.diff, self.layout = float(scale), float(eps), float(diff), layout
        self.q_width, self.k_width, self.v_width = heads * 2 * dim, kv_heads * 2 * dim, kv_heads * vdim
        self.w_in = nn.Parameter(torch.zeros(self.q_width + self.k_width + self.v_width + heads, hidden,
                                             dtype=dtype))                       # [q; k; v; gate]
        self.lq1 = nn.Parameter(torch.zeros(dim, dtype=torch.float32))
        self.lk1 = nn.Parameter(torch.zeros(dim, dtype=torch.float32))
        self.lq2 = nn.Parameter(torch.zeros(dim, dtype=torch.float32))
        self.lk2 = nn.Parameter(torch.zeros(dim, dtype=torch.float32))
        self.w_out = nn.Parameter(torch.zeros(hidden, heads * vdim, dtype=dtype))
        self.register_buffer("freqs", R.scaled_freqs(rot_dims, rot_base, rot_scaling), persistent=False)
        self._lam: Optional[torch.Tensor] = None      # [1] fp32 on the weights' device, formed on first use

    def cache_spec(self, name: str, page: int = 64):
        return {name: self.k_width + self.v_width}

    def lam(self) -> torch.Tensor:
        """exp(lq1 . lk1) - exp(lq2 . lk2) + diff, kept on the device (no host read in a step);
        call ``reset_lam`` after changing the four vectors."""
        if self._lam is None or self._lam.device != self.lq1.device:
            with torch.no_grad():
                self._lam = (torch.exp((self.lq1.float() * self.lk1.float()).sum())
                             - torch.exp((self.lq2.float() * self.lk2.float()).sum()) + self.diff).reshape(1)
        return self._lam

    def reset_lam(self):
        self._lam = None

    def forward(self, h: torch.Tensor, ctx, name: str) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        q = R.rope_norm_store(proj, self.heads * 2, self.kv_heads * 2, self.dim, self.v_width, self.freqs,
                              self.layout, False, self.eps, ctx.pools[name], ctx.batch)
        gate = proj[:, self.q_width + self.k_width + self.v_width:]
        o = R.differential_attention(q, gate, self.lam(), self.diff, self.eps, ctx.pools[name], self.heads,
                                     self.kv_heads, self.dim, self.vdim, self.scale, ctx.batch)
        return F.linear(o, self.w_out)
