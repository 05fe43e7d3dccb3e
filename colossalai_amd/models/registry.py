"""Model registry: pick a model class from a checkpoint folder's config.json.

A model class registers under the names a config can carry (``architecture``,
an entry of ``architectures`` or ``model_type``) and provides
``from_checkpoint(config_dict, tensors, dtype, device)``. ``load_pretrained``
reads ``config.json`` + ``model.safetensors`` from a folder and returns the
built model; engines, the CLI and the trace replayer all go through it.
"""

import json
import os
from typing import Callable, Dict

import torch

__all__ = ["register_model", "model_class_for", "load_pretrained", "registered_models"]

_MODELS: Dict[str, type] = {}


def register_model(*names: str) -> Callable[[type], type]:
    def deco(cls):
        for n in names:
            _MODELS[n.lower()] = cls
        return cls

    return deco


def registered_models():
    return sorted(_MODELS)


def model_class_for(config: dict) -> type:
    keys = []
    if isinstance(config.get("architecture"), str):
        keys.append(config["architecture"])
    keys += [a for a in config.get("architectures") or [] if isinstance(a, str)]
    if isinstance(config.get("model_type"), str):
        keys.append(config["model_type"])
    for k in keys:
        if k.lower() in _MODELS:
            return _MODELS[k.lower()]
    raise KeyError(f"no registered model for config names {keys}; known: {registered_models()}")


def load_pretrained(folder: str, dtype=torch.bfloat16, device="cpu"):
    """Build the model a folder describes (config.json + model.safetensors)."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    cls = model_class_for(config)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cls.from_checkpoint(config, tensors, dtype=dtype, device=device)
