"""MLP (dense feed-forward) with fused gated activation.

Capability analog of reference megatron/core/transformer/mlp.py:
fc1 column-parallel (doubled width for gated activations) -> fused
SwiGLU/GeGLU HIP kernel (K5) -> fc2 row-parallel.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from megatron_amd import ops
from megatron_amd.parallel.layers import ColumnParallelLinear, RowParallelLinear


class MLP(nn.Module):
    def __init__(self, config, is_expert: bool = False, ffn_hidden_size: int = None):
        super().__init__()
        self.config = config
        ffn = ffn_hidden_size if ffn_hidden_size is not None else config.ffn_hidden_size
        self.gated = config.activation in ("swiglu", "geglu")
        fc1_out = 2 * ffn if self.gated else ffn
        self.linear_fc1 = ColumnParallelLinear(
            config.hidden_size, fc1_out, config=config, bias=config.add_linear_bias, is_expert=is_expert
        )
        self.linear_fc2 = RowParallelLinear(
            ffn, config.hidden_size, config=config, bias=config.add_linear_bias, is_expert=is_expert
        )
        if self.gated:
            # per-TP-rank layout is [gate_shard ; up_shard]: checkpointing must
            # split this weight into two global tensors to be reshard-safe
            self.linear_fc1.weight.is_gated_fc1 = True
        self.activation = config.activation

    def _act(self, x: torch.Tensor) -> torch.Tensor:
        if self.activation == "swiglu":
            return ops.swiglu(x)
        if self.activation == "geglu":
            return ops.geglu(x)
        if self.activation == "gelu":
            return torch.nn.functional.gelu(x)
        if self.activation == "squared_relu":
            return ops.squared_relu(x)
        raise ValueError(self.activation)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        h, _ = self.linear_fc1(hidden_states)
        if self.gated:
            # column-parallel sharding keeps [x1_shard | x2_shard] adjacency per rank:
            # fc1 weight rows are [ffn/tp gate rows ; ffn/tp up rows] interleaved per rank
            h = self._act(h)
        else:
            h = self._act(h)
        out, _ = self.linear_fc2(h)
        return out


class XieluMLP(nn.Module):
    """Dense two-matrix feed-forward with the xIELU activation
    (ops.ragged.xielu): for z > 0, softplus(p) z^2 + z/2; otherwise
    (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2, with two learned raw scalars
    ``act = (p, q)``.  Plain replicated weights (serving path)."""

    def __init__(self, hidden: int, ffn: int, dtype=torch.bfloat16):
        super().__init__()
        self.w_up = nn.Parameter(torch.zeros(ffn, hidden, dtype=dtype))
        self.w_down = nn.Parameter(torch.zeros(hidden, ffn, dtype=dtype))
        self.act = nn.Parameter(torch.zeros(2, dtype=torch.float32))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        import torch.nn.functional as F

        from megatron_amd.ops import ragged as R

        return F.linear(R.xielu(F.linear(h, self.w_up), self.act, h.dtype), self.w_down)


class GeluMLP(nn.Module):
    """Dense two-matrix feed-forward without biases, activation = the tanh form
    of GELU (ops.ragged.gelu_tanh).  Plain replicated weights (serving path)."""

    def __init__(self, hidden: int, ffn: int, dtype=torch.bfloat16):
        super().__init__()
        self.w_up = nn.Parameter(torch.zeros(ffn, hidden, dtype=dtype))
        self.w_down = nn.Parameter(torch.zeros(hidden, ffn, dtype=dtype))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        import torch.nn.functional as F

        from megatron_amd.ops import ragged as R

        return F.linear(R.gelu_tanh(F.linear(h, self.w_up), h.dtype), self.w_down)


class GeluGLUMLP(nn.Module):
    """Dense gated feed-forward without biases, down(gelu_tanh(gate h) * (up h));
    [gate; up] is one matrix (ops.ragged.glu, kind "gelu_tanh").  Plain replicated
    weights (serving path)."""

    def __init__(self, hidden: int, ffn: int, dtype=torch.bfloat16):
        super().__init__()
        self.w_gate_up = nn.Parameter(torch.zeros(2 * ffn, hidden, dtype=dtype))
        self.w_down = nn.Parameter(torch.zeros(hidden, ffn, dtype=dtype))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        import torch.nn.functional as F

        from megatron_amd.ops import ragged as R

        return F.linear(R.glu(F.linear(h, self.w_gate_up), "gelu_tanh", 0.0, 0.0, h.dtype), self.w_down)
