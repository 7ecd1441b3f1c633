"""Grouped-query softmax attention whose weights are mixed over the heads after
the softmax (talking heads), restricted to chunks of the sequence.

Per token, from one fused projection with bias [q | k | v]:
  * every head of q and of k is divided by its own root mean square and scaled
    by a weight of the head size that all heads share,
  * the first ``rot_dims`` entries of every q and k head are rotated in
    neighbouring pairs (2i, 2i+1) by the angle position * rot_base^(-2i/rot_dims);
    the other entries pass unchanged,
  * ``value_mix``: v <- (1 - lam) v + lam v_first, v_first being the values the
    first such layer of the model computed for the same token (that layer keeps
    its own values); the mixed values are what the cache holds,
  * score_g(i, j) = q_g(i) . k_kv(g)(j) * scale * temp[g]; position i sees
    j <= i in its own chunk of ``chunk`` positions counted from the start of
    the sequence (chunk None: every j <= i); P_g = softmax_j score_g,
  * o_h(i) = sum_j (sum_g talk[h, g] P_g(i, j)) v_kv(h)(j): head h applies the
    mixed weights to the values of its own key/value head,
  * output projection with bias over the concatenated heads.

Cache: one paged pool of a HybridInferenceContext, rows [k | v] per token
(k normed and rotated, v mixed).  The step's own rows are written before
attention, so whole prompts, portions and decoded tokens are one path.  Values
of the first mixing layer travel to the later ones through ``carry``, a dict
that lives for one step (they are of the step's own tokens).

Scores, softmax, the head mixing and the weighted sums are fp32
(ops.ragged.talking_attention)."""

from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class TalkingHeadsAttention(nn.Module):
    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, eps: float,
                 rot_dims: int = 0, rot_base: float = 10000.0, chunk: Optional[int] = None,
                 value_mix: bool = False, dtype=torch.bfloat16):
        super().__init__()
        assert heads % kv_heads == 0, "query heads are a multiple of key/value heads"
        assert rot_dims % 2 == 0 and 0 <= rot_dims <= dim, "rotated entries come in pairs inside a head"
        assert chunk is None or chunk >= 1
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.eps, self.chunk, self.value_mix = float(scale), float(eps), chunk, bool(value_mix)
        self.q_width, self.k_width, self.v_width = heads * dim, kv_heads * dim, kv_heads * vdim
        rows = self.q_width + self.k_width + self.v_width
        self.w_in = nn.Parameter(torch.zeros(rows, hidden, dtype=dtype))          # [q; k; v]
        self.b_in = nn.Parameter(torch.zeros(rows, dtype=dtype))
        self.q_norm = nn.Parameter(torch.ones(dim, dtype=torch.float32))
        self.k_norm = nn.Parameter(torch.ones(dim, dtype=torch.float32))
        self.temp = nn.Parameter(torch.ones(heads, dtype=torch.float32))
        self.talk = nn.Parameter(torch.eye(heads, dtype=torch.float32))
        self.lam = nn.Parameter(torch.zeros(1, dtype=torch.float32))
        self.w_out = nn.Parameter(torch.zeros(hidden, heads * vdim, dtype=dtype))
        self.b_out = nn.Parameter(torch.zeros(hidden, dtype=dtype))
        self.register_buffer("freqs", R.pair_freqs(rot_dims, rot_base), persistent=False)

    def cache_spec(self, name: str, page: int = 64):
        return {name: self.k_width + self.v_width}

    def state_spec(self, name: str):
        return {}

    def forward(self, h: torch.Tensor, ctx, name: str, carry: dict) -> torch.Tensor:
        proj = F.linear(h, self.w_in, self.b_in)
        v_first = None
        if self.value_mix:
            v_first = carry.get("v_first")
            if v_first is None:
                carry["v_first"] = proj[:, self.q_width + self.k_width:]
            else:
                assert v_first.shape[1] == self.v_width, "layers that mix values share the value width"
        q = R.head_norm_rope_store(proj, self.heads, self.kv_heads, self.dim, self.vdim, self.q_norm, self.k_norm,
                                   self.eps, self.freqs, v_first, self.lam, ctx.pools[name], ctx.batch)
        o = R.talking_attention(q, ctx.pools[name], self.heads, self.kv_heads, self.dim, self.vdim, self.scale,
                                self.temp, self.talk, self.chunk or 0, ctx.batch, h.dtype)
        return F.linear(o, self.w_out, self.b_out)
