"""Tilarax: a decoder-only LM that stacks, in the order its config.json gives,
chunked talking-heads attention layers (per-head q/k norm, partial pairwise
rotation, per-head temperature, value mixing with the first such layer) and
mLSTM layers, each followed by a dense tanh-GELU or a routed SiLU-GLU
feed-forward (or none).

Sublayers read the residual stream itself and are normed on their OUTPUT:

    x <- x + norm1(mixer(x));   x <- x + norm2(ff(x)),   norm(y) = y / rms(y) * (1 + w)

and what a layer hands on is a learned weighted sum over depth: with X_0 the
embedding output and X_(i+1) the result of layer i,
x <- sum_{j <= i+1} dwa_i[j] X_j.  The embedding matrix is also the output
matrix; the model's norm before it has the same (1 + w) form.

The model only has a ragged forward (see models/bezutar.py): a flat batch of
tokens laid out by the engine's cache/state manager.  Sizes, layer order and
every constant come from config.json.  The residual, the depth history, norms,
routers, scores and recurrent state are fp32 in every compute dtype.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.models.bezutar import InferenceSpec
from megatron_amd.moe.routed_experts import RoutedExpertsMLP
from megatron_amd.ops import ragged as R
from megatron_amd.ssm.mlstm import MLSTMMixer
from megatron_amd.transformer.mlp import GeluMLP
from megatron_amd.transformer.talking_heads_attention import TalkingHeadsAttention


@dataclass
class TilaraxConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: List[dict]
    params_dtype: torch.dtype = torch.bfloat16
    max_position_embeddings: Optional[int] = None   # rotation angles are computed, not tabulated: no limit
    raw: dict = field(default_factory=dict, repr=False)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict, dtype=torch.bfloat16) -> "TilaraxConfig":
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   layers=list(d["layers"]), params_dtype=dtype, raw=d)


class TilaraxLayer(nn.Module):
    def __init__(self, cfg: TilaraxConfig, index: int):
        super().__init__()
        spec = cfg.layers[index]
        m = spec["mixer"]
        W, dt, eps = cfg.hidden_size, cfg.params_dtype, cfg.norm_eps
        self.kind = spec["type"]
        self.name = f"l{index}"
        if self.kind == "attention":
            rot, mask = m.get("rot") or {}, m.get("mask") or {}
            self.mixer = TalkingHeadsAttention(
                W, int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]),
                float(m["scale"]), eps, rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                chunk=int(mask["size"]) if mask.get("size") else None, value_mix=bool(m.get("v_mix", False)), dtype=dt)
        elif self.kind == "mlstm":
            self.mixer = MLSTMMixer(W, int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"]), eps,
                                    f"l{index}.mlstm", dtype=dt)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.norm1 = nn.Parameter(torch.zeros(W, dtype=torch.float32))            # applied as 1 + w
        mlp = spec.get("mlp")
        if mlp:
            kind = mlp.get("kind", "dense")
            if kind == "dense":
                self.mlp = GeluMLP(W, int(mlp["ff"]), dtype=dt)
            elif kind == "moe":
                ro = mlp["router"]
                self.mlp = RoutedExpertsMLP(W, int(ro["experts"]), int(ro["top"]), int(mlp["expert"]["ff"]), 0.0,
                                            score="softmax", router_bias=True, activation="silu", dtype=dt)
            else:
                raise ValueError(f"unknown feed-forward kind {kind!r}")
            self.norm2 = nn.Parameter(torch.zeros(W, dtype=torch.float32))
        else:
            self.mlp, self.norm2 = None, None
        self.dwa = nn.Parameter(torch.zeros(index + 2, dtype=torch.float32))      # weights of X_0 .. X_(index+1)

    def mix(self, h, ctx, carry):
        if self.kind == "attention":
            return self.mixer(h, ctx, self.name, carry)
        return self.mixer(h, ctx)


class TilaraxModel(nn.Module):
    ragged_batch = True                  # the engine schedules mixed prefill/decode steps for this model
    native_extensions = ("talking",)     # what a serving process has to build for it (ops/ragged.py)

    def __init__(self, config: TilaraxConfig):
        super().__init__()
        self.config = config
        W, dt = config.hidden_size, config.params_dtype
        self.embedding = nn.Parameter(torch.zeros(config.vocab_size, W, dtype=dt))   # also the output matrix
        self.layers = nn.ModuleList([TilaraxLayer(config, i) for i in range(config.num_layers)])
        self.final_norm_weight = nn.Parameter(torch.zeros(W, dtype=torch.float32))   # applied as 1 + w
        self.register_buffer("_one", torch.ones(1, dtype=torch.float32), persistent=False)
        self.layer_trace: Optional[list] = None   # debugging: what every layer hands on

    # -- what the cache/state manager must provide ------------------------------

    def inference_spec(self, page: int = 64) -> InferenceSpec:
        caches, states = {}, {}
        for layer in self.layers:
            if layer.kind == "attention":
                caches.update(layer.mixer.cache_spec(layer.name, page))
            else:
                states.update(layer.mixer.state_spec())
        return InferenceSpec(caches, states)

    # -- forward ------------------------------------------------------------------

    def forward_ragged(self, tokens: torch.Tensor, ctx, want: Optional[torch.Tensor] = None) -> torch.Tensor:
        """tokens [T] laid out by ctx.batch -> logits fp32 [len(want) or T, vocab]."""
        cfg = self.config
        dt, eps, L = cfg.params_dtype, cfg.norm_eps, cfg.num_layers
        x = R.embed_plain(tokens, self.embedding)                  # [T, W] fp32 residual
        hist = torch.empty(L + 1, *x.shape, dtype=torch.float32, device=x.device)
        h = R.post_norm_add(x, None, None, eps, dt, hist, 0, self._one)   # X_0 into the history, x in the GEMM dtype
        carry: dict = {}                                           # lives for this step (first mixed values)
        for i, layer in enumerate(self.layers):
            y = layer.mix(h, ctx, carry)
            if layer.mlp is not None:
                h = R.post_norm_add(x, y, layer.norm1, eps, dt)
                y = layer.mlp(h)
                h = R.post_norm_add(x, y, layer.norm2, eps, dt, hist, i + 1, layer.dwa)
            else:
                h = R.post_norm_add(x, y, layer.norm1, eps, dt, hist, i + 1, layer.dwa)
            if self.layer_trace is not None:
                self.layer_trace.append(x.clone())
        if want is not None:
            x = x.index_select(0, want)
        h, _ = R.residual_group_norm(x, None, self._final_scale(), None, 1, eps, dt)
        return F.linear(h, self.embedding).float()

    def _final_scale(self) -> torch.Tensor:
        return 1.0 + self.final_norm_weight.detach()

    def forward(self, input_ids: torch.Tensor, inference_context=None, want=None) -> torch.Tensor:
        """[b, s] ids -> logits [s, b, vocab] from empty caches and states (the
        call shape of the framework's other causal LMs); with an
        inference_context whose batch is laid out, ids are the flat tokens."""
        if inference_context is not None:
            return self.forward_ragged(input_ids.reshape(-1), inference_context, want)
        from megatron_amd.inference.contexts import HybridInferenceContext

        b, s = input_ids.shape
        bs = 64
        spec = self.inference_spec(bs)
        per = (s + bs - 1) // bs
        ctx = HybridInferenceContext(spec.caches, spec.states, b * per, bs, b,
                                     dtype=self.config.params_dtype, device=input_ids.device)
        tables = [ctx.allocator.allocate(per) for _ in range(b)]
        ctx.begin_batch([s] * b, [0] * b, [ctx.acquire_slot() for _ in range(b)], tables)
        logits = self.forward_ragged(input_ids.reshape(-1), ctx)
        return logits.view(b, s, -1).transpose(0, 1)


# ---------------------------------------------------------------------------
# weights: checkpoint tensor names -> module parameters
# ---------------------------------------------------------------------------


def load_tilarax_state(model: TilaraxModel, tensors: Dict[str, torch.Tensor]) -> None:
    """Copy a checkpoint's tensors (name -> tensor, Linear weights [out, in])
    into the model, fusing the projections that run as one GEMM."""
    used = set()

    def get(name):
        used.add(name)
        return tensors[name]

    with torch.no_grad():
        model.embedding.data.copy_(get("embed"))
        for i, layer in enumerate(model.layers):
            p = f"l{i}."
            a = p + "mix."
            mx = layer.mixer
            layer.norm1.data.copy_(get(p + "norm1"))
            if layer.kind == "attention":
                mx.w_in.data.copy_(torch.cat([get(a + "q"), get(a + "k"), get(a + "v")], dim=0))
                mx.b_in.data.copy_(torch.cat([get(a + "q.b"), get(a + "k.b"), get(a + "v.b")], dim=0))
                mx.q_norm.data.copy_(get(a + "q.norm"))
                mx.k_norm.data.copy_(get(a + "k.norm"))
                mx.temp.data.copy_(get(a + "temp"))
                mx.talk.data.copy_(get(a + "talk"))
                if a + "vmix" in tensors:                       # the first mixing layer never reads its own
                    mx.lam.data.copy_(get(a + "vmix").reshape(1))
                mx.w_out.data.copy_(get(a + "o"))
                mx.b_out.data.copy_(get(a + "o.b"))
            else:
                mx.w_in.data.copy_(torch.cat([get(a + "q"), get(a + "k"), get(a + "v"), get(a + "g")], dim=0))
                mx.w_gates.data.copy_(torch.cat([get(a + "i"), get(a + "f")], dim=0))
                mx.bias_i.data.copy_(get(a + "i.b"))
                mx.bias_f.data.copy_(get(a + "f.b"))
                mx.norm_weight.data.copy_(get(a + "norm"))
                mx.w_out.data.copy_(get(a + "o"))
            if layer.mlp is not None:
                ff, q = layer.mlp, p + "mlp."
                layer.norm2.data.copy_(get(p + "norm2"))
                if isinstance(ff, GeluMLP):
                    ff.w_up.data.copy_(get(q + "up"))
                    ff.w_down.data.copy_(get(q + "down"))
                else:
                    ff.w_router.data.copy_(get(q + "router"))
                    ff.b_router.data.copy_(get(q + "router.b"))
                    for e in range(ff.experts):
                        ff.w_gate_up.data[e].copy_(torch.cat([get(f"{q}e{e}.gate"), get(f"{q}e{e}.up")], dim=0))
                        ff.w_down.data[e].copy_(get(f"{q}e{e}.down"))
            layer.dwa.data.copy_(get(p + "dwa"))
        model.final_norm_weight.data.copy_(get("final.norm"))
    unused = set(tensors) - used
    if unused:
        import warnings

        warnings.warn(f"checkpoint tensors without a place in the model are ignored: {sorted(unused)[:8]}")


def build_tilarax_from_dir(path: str, dtype=torch.bfloat16, device="cpu") -> TilaraxModel:
    from safetensors import safe_open

    with open(os.path.join(path, "config.json")) as f:
        cfg = TilaraxConfig.from_dict(json.load(f), dtype=dtype)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as f:
        for k in f.keys():
            tensors[k] = f.get_tensor(k)
    model = TilaraxModel(cfg)
    load_tilarax_state(model, tensors)
    return model.to(device).eval()
