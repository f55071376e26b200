"""Architecture registry: a checkpoint folder's ``config.json`` names the
model class, the way ``init_inference`` users expect from Hugging Face style
folders.

``register_architecture(name, build)`` adds a builder
``build(config_dict, dtype) -> nn.Module`` (with ``wants_tensors=True`` it is
called as ``build(config_dict, dtype, tensors)`` so sizes that only tensor
shapes give can be read; ``tensors`` is None without a checkpoint); the module may define
``load_named_tensors(dict)`` to take checkpoint tensors under their file
names (otherwise ``load_state_dict`` is used). ``load_pretrained(folder)``
reads config.json + *.safetensors and returns the model on ``device``.
"""

import glob
import json
import os
from dataclasses import fields
from typing import Callable, Dict

import torch

_BUILDERS: Dict[str, Callable] = {}
_WANTS_TENSORS = set()


def register_architecture(name: str, build: Callable,
                          wants_tensors: bool = False):
    _BUILDERS[name] = build
    if wants_tensors:
        _WANTS_TENSORS.add(name)
    else:
        _WANTS_TENSORS.discard(name)


def architectures():
    return sorted(_BUILDERS)


def _arch_name(cfg: dict) -> str:
    name = cfg.get("architecture")
    if name is None and cfg.get("architectures"):
        name = cfg["architectures"][0]
    if name is None:
        raise ValueError("config.json names no architecture")
    return name


def build_model(cfg: dict, dtype=torch.bfloat16, tensors=None):
    name = _arch_name(cfg)
    if name not in _BUILDERS:
        raise ValueError(f"unknown architecture {name!r}; known: "
                         f"{architectures()}")
    if name in _WANTS_TENSORS:
        return _BUILDERS[name](cfg, dtype, tensors)
    return _BUILDERS[name](cfg, dtype)


def load_pretrained(folder: str, dtype=torch.bfloat16, device="cpu"):
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    for path in sorted(glob.glob(os.path.join(folder, "*.safetensors"))):
        tensors.update(load_file(path))
    if not tensors:
        raise FileNotFoundError(f"no *.safetensors under {folder}")
    model = build_model(cfg, dtype, tensors)
    if hasattr(model, "load_named_tensors"):
        model.load_named_tensors(tensors)
    else:
        model.load_state_dict(tensors, strict=False)
        model.to(dtype)
    return model.to(device).eval()


def _dataclass_builder(config_cls, model_cls, rename=None):
    """Builder for the dataclass-configured models: config.json keys that
    match a config field (after ``rename``) are taken, the rest ignored."""
    rename = rename or {}

    def build(cfg, dtype):
        names = {f.name for f in fields(config_cls)}
        kw = {rename.get(k, k): v for k, v in cfg.items()}
        model = model_cls(config_cls(**{k: v for k, v in kw.items()
                                        if k in names}))
        return model.to(dtype)
    return build


def _register_builtin():
    from .fizesun import FizesunConfig, FizesunForCausalLM
    from .llama import LlamaConfig, LlamaForCausalLM
    from .lolulorn import build_from_config as build_lolulorn
    from .mixtral import MixtralConfig, MixtralForCausalLM
    from .numolorn import build_from_config as build_numolorn
    from .savovik import build_from_config as build_savovik
    hf = {"num_hidden_layers": "num_layers",
          "num_attention_heads": "num_heads",
          "num_key_value_heads": "num_kv_heads",
          "max_position_embeddings": "max_seq_len",
          "rms_norm_eps": "rms_eps",
          "num_local_experts": "num_experts",
          "num_experts_per_tok": "top_k"}
    register_architecture("LlamaForCausalLM",
                          _dataclass_builder(LlamaConfig, LlamaForCausalLM, hf))
    register_architecture("MixtralForCausalLM",
                          _dataclass_builder(MixtralConfig,
                                             MixtralForCausalLM, hf))
    register_architecture(
        "Fizesun", lambda cfg, dtype: FizesunForCausalLM(
            FizesunConfig.from_dict(cfg), dtype))
    register_architecture("Lolulorn", build_lolulorn, wants_tensors=True)
    register_architecture("Savovik", build_savovik)
    register_architecture("Numolorn", build_numolorn, wants_tensors=True)


_register_builtin()
