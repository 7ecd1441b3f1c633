"""Model registry: architecture name (config.json) -> builder.

A served model directory holds config.json and weights; ``build_from_dir``
reads the architecture name (key "architecture", or the first entry of the
HuggingFace-style "architectures") and calls the registered builder, which
returns an eval-mode module on the requested device and dtype.
"""

from __future__ import annotations

import json
import os
from typing import Callable, Dict

import torch

_BUILDERS: Dict[str, Callable] = {}


def register_model(name: str):
    def deco(fn):
        _BUILDERS[name] = fn
        return fn

    return deco


def registered_models():
    return sorted(_BUILDERS)


def architecture_of(path: str) -> str:
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    name = cfg.get("architecture") or (cfg.get("architectures") or [None])[0]
    if name is None:
        raise ValueError(f"{path}/config.json names no architecture")
    return name


def build_from_dir(path: str, dtype=torch.bfloat16, device="cpu"):
    name = architecture_of(path)
    if name not in _BUILDERS:
        raise ValueError(f"unknown architecture {name!r}; registered: {registered_models()}")
    return _BUILDERS[name](path, dtype=dtype, device=device)


@register_model("Bezutar")
def _bezutar(path, dtype, device):
    from megatron_amd.models.bezutar import build_bezutar_from_dir

    return build_bezutar_from_dir(path, dtype=dtype, device=device)


@register_model("Bezurax")
def _bezurax(path, dtype, device):
    from megatron_amd.models.bezurax import build_bezurax_from_dir

    return build_bezurax_from_dir(path, dtype=dtype, device=device)


@register_model("Tilarax")
def _tilarax(path, dtype, device):
    from megatron_amd.models.tilarax import build_tilarax_from_dir

    return build_tilarax_from_dir(path, dtype=dtype, device=device)


@register_model("Lomazen")
def _lomazen(path, dtype, device):
    from megatron_amd.models.lomazen import build_lomazen_from_dir

    return build_lomazen_from_dir(path, dtype=dtype, device=device)


@register_model("LlamaForCausalLM")
def _llama(path, dtype, device):
    """HuggingFace Llama checkpoints -> GPTModel (single process, TP=1)."""
    from megatron_amd.config import TransformerConfig
    from megatron_amd.models.gpt import GPTModel
    from megatron_amd.parallel import grid as G

    with open(os.path.join(path, "config.json")) as f:
        hf = json.load(f)
    if not G.grid_initialized():
        G.initialize_model_parallel(world_size=1, rank=0)
    cfg = TransformerConfig(
        num_layers=hf["num_hidden_layers"], hidden_size=hf["hidden_size"],
        num_attention_heads=hf["num_attention_heads"],
        num_query_groups=hf.get("num_key_value_heads", hf["num_attention_heads"]),
        ffn_hidden_size=hf["intermediate_size"], vocab_size=hf["vocab_size"],
        max_position_embeddings=hf.get("max_position_embeddings", 4096),
        rotary_base=hf.get("rope_theta", 10000.0), layernorm_epsilon=hf.get("rms_norm_eps", 1e-5),
        untie_embeddings_and_output_weights=not hf.get("tie_word_embeddings", False),
        bf16=dtype == torch.bfloat16)
    import importlib.util
    import sys

    repo = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    spec = importlib.util.spec_from_file_location(
        "_convert_hf", os.path.join(repo, "tools", "checkpoint", "convert_hf.py"))
    conv = importlib.util.module_from_spec(spec)
    sys.modules["_convert_hf"] = conv
    spec.loader.exec_module(conv)
    from safetensors.torch import load_file

    sd = {}
    for fn in sorted(os.listdir(path)):
        if fn.endswith(".safetensors"):
            sd.update(load_file(os.path.join(path, fn)))
    model = GPTModel(cfg)
    model.load_state_dict(conv.hf_to_mcore_state_dict(sd, cfg), strict=False)
    return model.to(device=device, dtype=dtype).eval()
