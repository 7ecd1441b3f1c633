"""Lomazen: a decoder-only LM that stacks, in the order its config.json gives,
two kinds of attention layers,

  * "attention": grouped-query attention whose q and k are rotated in
    neighbouring pairs (frequencies optionally rescaled by wavelength) and then
    unit-normed per head, with capped scores and an elementwise sigmoid gate
    (transformer/gated_softcap_attention.py),
  * "attention_2": differential attention, two softmax maps a head over the same
    values, rotated in halves, with one gate per head
    (transformer/differential_attention.py),

each followed by a dense GELU-GLU feed-forward, routed squared-ReLU experts
weighted by their softmax score over all experts, or nothing.  Sublayers are
normed on both sides:

    x <- x + norm1b(mixer(norm1(x)));   x <- x + norm2b(ff(norm2(x)))

A block of layers ``loop.start .. loop.stop - 1`` runs ``loop.times`` times in a
row with the same weights; every pass has its own cache pools.  Right before a
pass, x <- W_in [x; x0] + step[pass], x0 being the embedding output.  The
embedding matrix is the output matrix, logits are scaled by ``logit_scale``.

The model only has a ragged forward (see models/bezutar.py): a flat batch of
tokens laid out by the engine's cache/state manager.  Sizes, layer order and
every constant come from config.json.  The residual, norms, routers, angles,
scores and softmax are fp32 in every compute dtype.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from megatron_amd.models.bezutar import InferenceSpec
from megatron_amd.moe.routed_experts import RoutedExpertsMLP
from megatron_amd.ops import ragged as R
from megatron_amd.transformer.differential_attention import DifferentialAttention
from megatron_amd.transformer.gated_softcap_attention import GatedSoftcapAttention
from megatron_amd.transformer.mlp import GeluGLUMLP


@dataclass
class LomazenConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: List[dict]
    logit_scale: float = 1.0
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0                             # 0: no repeated block, no restart matrix
    params_dtype: torch.dtype = torch.bfloat16
    max_position_embeddings: Optional[int] = None   # rotation angles are computed, not tabulated: no limit
    raw: dict = field(default_factory=dict, repr=False)

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict, dtype=torch.bfloat16) -> "LomazenConfig":
        loop = d.get("loop") or {}
        cfg = cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                  layers=list(d["layers"]), logit_scale=float(d.get("logit_scale", 1.0)),
                  loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                  loop_times=int(loop.get("times", 0)) if loop else 0, params_dtype=dtype, raw=d)
        if cfg.loop_times:
            assert 0 <= cfg.loop_start < cfg.loop_stop <= cfg.num_layers, "the repeated block lies inside the stack"
        return cfg

    def runs(self) -> List[Tuple[int, int, bool]]:
        """(layer, pass, first of its pass) for every layer run of a forward."""
        n = self.num_layers
        if not self.loop_times:
            return [(i, 0, False) for i in range(n)]
        out = [(i, 0, False) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            out += [(i, t, i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        out += [(i, 0, False) for i in range(self.loop_stop, n)]
        return out


class LomazenLayer(nn.Module):
    def __init__(self, cfg: LomazenConfig, index: int):
        super().__init__()
        spec = cfg.layers[index]
        m = spec["mixer"]
        W, dt, eps = cfg.hidden_size, cfg.params_dtype, cfg.norm_eps
        self.kind = spec["type"]
        self.name = f"l{index}"
        rot = m.get("rot") or {}
        common = dict(rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                      rot_scaling=rot.get("scaling"), dtype=dt)
        heads, kv = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
        if self.kind == "attention":
            self.mixer = GatedSoftcapAttention(W, heads, kv, int(m["dim"]), int(m["vdim"]), float(m["scale"]), eps,
                                               softcap=m.get("softcap"), layout="pairs", unit_norm=True, **common)
        elif self.kind == "attention_2":
            self.mixer = DifferentialAttention(W, heads, kv, int(m["dim"]), int(m["vdim"]), float(m["scale"]), eps,
                                               float(m["diff"]), layout="halves", **common)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.norm1 = nn.Parameter(torch.ones(W, dtype=torch.float32))     # before the mixer
        self.norm1b = nn.Parameter(torch.ones(W, dtype=torch.float32))    # on the mixer's output
        mlp = spec.get("mlp")
        if mlp:
            kind = mlp.get("kind", "dense")
            if kind == "dense":
                self.mlp = GeluGLUMLP(W, int(mlp["ff"]), dtype=dt)
            elif kind == "moe":
                ro = mlp["router"]
                self.mlp = RoutedExpertsMLP(W, int(ro["experts"]), int(ro["top"]), int(mlp["expert"]["ff"]), 0.0,
                                            score="softmax_all", activation="relu2", dtype=dt)
            else:
                raise ValueError(f"unknown feed-forward kind {kind!r}")
            self.norm2 = nn.Parameter(torch.ones(W, dtype=torch.float32))
            self.norm2b = nn.Parameter(torch.ones(W, dtype=torch.float32))
        else:
            self.mlp, self.norm2, self.norm2b = None, None, None

    def pool_name(self, run: int, looped: bool) -> str:
        return f"{self.name}.p{run}" if looped else self.name


class LomazenModel(nn.Module):
    ragged_batch = True                  # the engine schedules mixed prefill/decode steps for this model
    native_extensions = ("gated",)       # what a serving process has to build for it (ops/ragged.py)

    def __init__(self, config: LomazenConfig):
        super().__init__()
        self.config = config
        W, dt = config.hidden_size, config.params_dtype
        self.embedding = nn.Parameter(torch.zeros(config.vocab_size, W, dtype=dt))   # also the output matrix
        self.layers = nn.ModuleList([LomazenLayer(config, i) for i in range(config.num_layers)])
        if config.loop_times:
            self.loop_in = nn.Parameter(torch.zeros(W, 2 * W, dtype=dt))             # applied to [x; x0]
            self.loop_step = nn.Parameter(torch.zeros(config.loop_times, W, dtype=torch.float32))
        self.final_norm_weight = nn.Parameter(torch.ones(W, dtype=torch.float32))
        self.layer_trace: Optional[list] = None   # debugging: the residual after every layer run

    # -- what the cache/state manager must provide ------------------------------

    def _looped(self, i: int) -> bool:
        c = self.config
        return bool(c.loop_times) and c.loop_start <= i < c.loop_stop

    def inference_spec(self, page: int = 64) -> InferenceSpec:
        caches = {}
        for i, t, _ in self.config.runs():
            layer = self.layers[i]
            caches.update(layer.mixer.cache_spec(layer.pool_name(t, self._looped(i)), page))
        return InferenceSpec(caches, {})

    # -- forward ------------------------------------------------------------------

    def forward_ragged(self, tokens: torch.Tensor, ctx, want: Optional[torch.Tensor] = None) -> torch.Tensor:
        """tokens [T] laid out by ctx.batch -> logits fp32 [len(want) or T, vocab]."""
        cfg = self.config
        dt, eps, W = cfg.params_dtype, cfg.norm_eps, cfg.hidden_size
        runs = cfg.runs()
        x = R.embed_plain(tokens, self.embedding)                  # [T, W] fp32 residual = x0
        xx = None
        if cfg.loop_times:
            # [x | x0] in the GEMM dtype: the right half is written once a step, the left before every pass
            xx = torch.empty(x.shape[0], 2 * W, dtype=dt, device=x.device)
            xx[:, W:].copy_(x)
        h = None                                                   # normed input of the next sublayer
        y = post = None                                            # a sublayer's output waiting for its norm + add
        for n, (i, t, first) in enumerate(runs):
            layer = self.layers[i]
            if first:
                # fold what is pending, hand x to the restart GEMM, start a fresh residual
                R.sandwich_norm_add(x, y, post, None, eps, dt, copy_to=xx[:, :W])
                x, h = R.restart_norm(F.linear(xx, self.loop_in), self.loop_step[t], layer.norm1, eps, dt)
            else:
                h = R.sandwich_norm_add(x, y, post, layer.norm1, eps, dt)
            y = layer.mixer(h, ctx, layer.pool_name(t, self._looped(i)))
            post = layer.norm1b
            if layer.mlp is not None:
                h = R.sandwich_norm_add(x, y, post, layer.norm2, eps, dt)
                y, post = layer.mlp(h), layer.norm2b
            if self.layer_trace is not None:
                R.sandwich_norm_add(x, y, post, None, eps, dt)
                y = post = None
                self.layer_trace.append(x.clone())
        R.sandwich_norm_add(x, y, post, None, eps, dt)
        if want is not None:
            x = x.index_select(0, want)
        h, _ = R.residual_group_norm(x, None, self.final_norm_weight, None, 1, eps, dt)
        logits = F.linear(h, self.embedding).float()
        return logits * cfg.logit_scale if cfg.logit_scale != 1.0 else logits

    def forward(self, input_ids: torch.Tensor, inference_context=None, want=None) -> torch.Tensor:
        """[b, s] ids -> logits [s, b, vocab] from empty caches (the call shape of
        the framework's other causal LMs); with an inference_context whose batch
        is laid out, ids are the flat tokens."""
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


def load_lomazen_state(model: LomazenModel, tensors: Dict[str, torch.Tensor]) -> None:
    """Copy a checkpoint's tensors (name -> tensor, Linear weights [out, in])
    into the model, fusing the projections that run as one GEMM."""
    used = set()

    def get(name):
        used.add(name)
        return tensors[name]

    with torch.no_grad():
        model.embedding.data.copy_(get("embed"))
        if model.config.loop_times:
            model.loop_in.data.copy_(get("loop.in"))
            model.loop_step.data.copy_(get("loop.step"))
        for i, layer in enumerate(model.layers):
            p = f"l{i}."
            a = p + "mix."
            mx = layer.mixer
            layer.norm1.data.copy_(get(p + "norm1"))
            layer.norm1b.data.copy_(get(p + "norm1b"))
            mx.w_in.data.copy_(torch.cat([get(a + "q"), get(a + "k"), get(a + "v"), get(a + "g")], dim=0))
            mx.w_out.data.copy_(get(a + "o"))
            if layer.kind == "attention_2":
                for nm in ("lq1", "lk1", "lq2", "lk2"):
                    getattr(mx, nm).data.copy_(get(a + nm))
                mx.reset_lam()
            if layer.mlp is not None:
                ff, q = layer.mlp, p + "mlp."
                layer.norm2.data.copy_(get(p + "norm2"))
                layer.norm2b.data.copy_(get(p + "norm2b"))
                if isinstance(ff, GeluGLUMLP):
                    ff.w_gate_up.data.copy_(torch.cat([get(q + "gate"), get(q + "up")], dim=0))
                    ff.w_down.data.copy_(get(q + "down"))
                else:
                    ff.w_router.data.copy_(get(q + "router"))
                    for e in range(ff.experts):
                        ff.w_up.data[e].copy_(get(f"{q}e{e}.up"))
                        ff.w_down.data[e].copy_(get(f"{q}e{e}.down"))
        model.final_norm_weight.data.copy_(get("final.norm"))
    unused = set(tensors) - used
    if unused:
        import warnings

        warnings.warn(f"checkpoint tensors without a place in the model are ignored: {sorted(unused)[:8]}")


def build_lomazen_from_dir(path: str, dtype=torch.bfloat16, device="cpu") -> LomazenModel:
    from safetensors import safe_open

    with open(os.path.join(path, "config.json")) as f:
        cfg = LomazenConfig.from_dict(json.load(f), dtype=dtype)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as f:
        for k in f.keys():
            tensors[k] = f.get_tensor(k)
    model = LomazenModel(cfg)
    load_lomazen_state(model, tensors)
    return model.to(device).eval()
