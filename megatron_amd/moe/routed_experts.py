"""Routed GLU experts for the ragged serving path (single process, all
experts resident; the training-side MoE with token dispatchers is
moe/moe_layer.py).

Router: logits in fp32, sigmoid scores, the ``top`` largest among the experts
of the best ``keep`` of ``groups`` neighbour groups (group score = sum of its
two largest scores; the selection rule of moe/router.py::group_limited_topk),
weights = chosen scores / their sum * route_scale.
Expert (no biases): g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
y = g sigmoid(alpha g) (u + 1), output W_down y.
Other designs choose by the raw logits and weigh by the softmax over the chosen
logits (``score="softmax"``, optional router bias), and use the plain SiLU GLU
y = g sigmoid(g) u (``activation="silu"``).  ``score="softmax_all"`` chooses the largest
logits and weighs them by their softmax over ALL experts (the weights do not
sum to one); ``activation="relu2"`` makes experts WITHOUT a gate matrix,
W_down relu(W_up h)^2 (``w_up`` [experts, ff, hidden] in place of ``w_gate_up``).
Optional shared expert of the same form for every token, times
sigmoid(w_sg . h); its gate row rides in the fp32 router GEMM.

Step: one router kernel (fp32 logits of [router; shared gate], scores, selection), then
  * many pairs (prompt portions): the (token, choice) pairs are sorted by expert;
    bf16 runs one grouped GEMM per linear over the sorted pairs with the group
    ends on the device (no host read); fp32 and unaligned sizes run each expert
    with work on its slice (vendor GEMMs; the pair counts are one host read),
  * few pairs (decoding): two kernels in which every pair streams its expert's
    matrices (ops.ragged.expert_pairs), no sort and no host read,
and one kernel forms sum_k weight_k down_k + sigmoid(gate) shared + add in fp32.
"""

from __future__ import annotations

import os
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.ops import ragged as R


class RoutedExpertsMLP(nn.Module):
    def __init__(self, hidden: int, experts: int, top: int, ff: int, limit: float, groups: int = 1,
                 keep: int = 1, route_scale: float = 1.0, shared_ff: Optional[int] = None,
                 shared_limit: Optional[float] = None, alpha: float = 1.702, score: str = "sigmoid",
                 router_bias: bool = False, activation: str = "clamped", dtype=torch.bfloat16):
        super().__init__()
        assert score in R.ROUTER_SCORES and (activation in R.GLU_KINDS or activation == "relu2")
        self.gated = activation != "relu2"
        assert self.gated or not shared_ff, "the shared expert is a GLU"
        assert score == "sigmoid" or groups <= 1, "group-limited choice is defined on sigmoid scores"
        self.score, self.activation = score, activation
        assert top <= experts and experts % max(groups, 1) == 0
        if groups > 1:
            assert keep * (experts // groups) >= top, "the kept groups hold fewer experts than are chosen"
        self.experts, self.top, self.ff, self.limit = experts, top, ff, float(limit)
        self.groups, self.keep, self.route_scale, self.alpha = max(groups, 1), keep, float(route_scale), float(alpha)
        self.shared_ff = shared_ff
        self.shared_limit = float(shared_limit) if shared_ff else None
        # row ``experts`` (when there is a shared expert) is its gate vector
        self.w_router = nn.Parameter(torch.zeros(experts + (1 if shared_ff else 0), hidden, dtype=torch.float32))
        self.b_router = (nn.Parameter(torch.zeros(experts + (1 if shared_ff else 0), dtype=torch.float32))
                         if router_bias else None)
        if self.gated:
            self.w_gate_up = nn.Parameter(torch.zeros(experts, 2 * ff, hidden, dtype=dtype))   # [gate; up] per expert
        else:
            self.w_up = nn.Parameter(torch.zeros(experts, ff, hidden, dtype=dtype))
        self.w_down = nn.Parameter(torch.zeros(experts, hidden, ff, dtype=dtype))
        if shared_ff:
            self.ws_gate_up = nn.Parameter(torch.zeros(2 * shared_ff, hidden, dtype=dtype))
            self.ws_down = nn.Parameter(torch.zeros(hidden, shared_ff, dtype=dtype))

    def route(self, h: torch.Tensor):
        """-> (ids [T, top], weights [T, top], the shared expert's gate logit [T, 1] or [T, 0])"""
        return R.moe_router(h, self.w_router, self.experts, self.top, self.groups, self.keep, self.route_scale,
                            self.b_router, self.score)

    def _glu(self, gu, limit, dtype):
        if not self.gated:
            return R.relu2(gu, dtype)
        return R.glu(gu, self.activation, limit, self.alpha, dtype)

    def _grouped_ok(self, h: torch.Tensor) -> bool:
        """bf16 on the GPU with 16-byte aligned rows: the grouped GEMM the training-side
        expert layer uses (ops.grouped_linear), here with its offsets left on the device."""
        return (h.is_cuda and h.dtype == torch.bfloat16 and hasattr(torch, "_grouped_mm")
                and h.shape[1] % 8 == 0 and self.ff % 8 == 0
                and os.environ.get("MEGATRON_AMD_NO_TORCH_GROUPED", "0") != "1")

    def forward(self, h: torch.Tensor, add: Optional[torch.Tensor] = None) -> torch.Tensor:
        """h [T, hidden] in the compute dtype -> fp32 [T, hidden] (+ add)."""
        T, K, E = h.shape[0], self.top, self.experts
        ids, weights, extra = self.route(h)
        shared = gate = None
        if self.shared_ff:
            sy = self._glu(F.linear(h, self.ws_gate_up), self.shared_limit, h.dtype)
            shared = F.linear(sy, self.ws_down)
            gate = extra.reshape(-1)
        if R.expert_pairs_ok(h, K, self.ff):
            # few pairs (decoding): each pair streams its expert's matrices, no sort, no host read
            if self.gated:
                down = R.expert_pairs(h, ids, self.w_gate_up, self.w_down, self.limit, self.alpha, self.activation)
            else:
                down = R.expert_pairs_plain(h, ids, self.w_up, self.w_down)
            inv = torch.arange(T * K, dtype=torch.int32, device=h.device).view(T, K)
            return R.moe_combine(down, inv, weights, shared, gate, add)
        flat = ids.reshape(-1).long()
        order = torch.argsort(flat, stable=True)              # pairs sorted by expert
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=order.device)
        xs = h.index_select(0, torch.div(order, K, rounding_mode="floor"))
        w_first = self.w_gate_up if self.gated else self.w_up
        down = None
        if self._grouped_ok(h) and not getattr(self, "_grouped_refused", False):
            # one grouped GEMM per linear over the sorted pairs, group ends on the device: no host read
            offs = torch.cumsum(torch.bincount(flat, minlength=E), 0).to(torch.int32)
            try:
                gu = torch._grouped_mm(xs, w_first.transpose(1, 2), offs=offs)
                down = torch._grouped_mm(self._glu(gu, self.limit, h.dtype),
                                         self.w_down.transpose(1, 2), offs=offs)
            except RuntimeError as e:          # a shape the vendor's grouped GEMM does not take
                import warnings

                warnings.warn(f"grouped GEMM refused these expert sizes ({e}); one GEMM per expert instead")
                self._grouped_refused = True
        if down is None:
            counts = torch.bincount(flat, minlength=E).tolist()   # the step's host read
            down = torch.empty(T * K, h.shape[1], dtype=h.dtype, device=h.device)
            at = 0
            for e, n in enumerate(counts):
                if n:
                    gu = F.linear(xs[at:at + n], w_first[e])
                    down[at:at + n] = F.linear(self._glu(gu, self.limit, h.dtype), self.w_down[e])
                    at += n
        return R.moe_combine(down, inv.view(T, K).to(torch.int32), weights, shared, gate, add)
