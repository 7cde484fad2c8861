"""Model registry: which config / model class serves a checkpoint directory.

A directory's ``config.json`` names its architecture by ``architecture`` (layer-list checkpoints) or ``model_type``
(HF-style LLaMA configs; absent = LLaMA). ``load_model`` builds the model on a device in a number format and loads the
weights it finds there.
"""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, Tuple

import torch


def _llama():
    from ..config import LLaMAConfig
    from .llama import LLaMAForCausalLM
    return LLaMAConfig, LLaMAForCausalLM


def _zavevik():
    from ..config import ZavevikConfig
    from .zavevik import ZavevikForCausalLM
    return ZavevikConfig, ZavevikForCausalLM


def _zasevik():
    from ..config import ZasevikConfig
    from .zasevik import ZasevikForCausalLM
    return ZasevikConfig, ZasevikForCausalLM


def _besulix():
    from ..config import BesulixConfig
    from .besulix import BesulixForCausalLM
    return BesulixConfig, BesulixForCausalLM


def _zifisun():
    from ..config import ZifisunConfig
    from .zifisun import ZifisunForCausalLM
    return ZifisunConfig, ZifisunForCausalLM


# architecture name (lower case) -> () -> (config class, model class)
MODEL_REGISTRY: Dict[str, Callable[[], Tuple[type, type]]] = {"llama": _llama, "zavevik": _zavevik,
                                                              "zasevik": _zasevik, "besulix": _besulix,
                                                              "zifisun": _zifisun}
# families on the layer-list step function (models/layer_list.py): both number formats, the hybrid extension
LAYER_LIST_FAMILIES = ("zavevik", "zasevik", "besulix", "zifisun")


def register(name: str, factory: Callable[[], Tuple[type, type]]) -> None:
    MODEL_REGISTRY[name.lower()] = factory


def architecture_of(directory: str) -> str:
    with open(os.path.join(directory, "config.json")) as f:
        d = json.load(f)
    name = str(d.get("architecture") or d.get("model_type") or "llama").lower()
    if name not in MODEL_REGISTRY:
        raise KeyError(f"unknown architecture {name!r}; known: {sorted(MODEL_REGISTRY)}")
    return name


def resolve(directory: str) -> Tuple[str, type, type]:
    name = architecture_of(directory)
    cfg_cls, model_cls = MODEL_REGISTRY[name]()
    return name, cfg_cls, model_cls


def supports_dtype(name: str, dtype: torch.dtype) -> bool:
    """Number formats a family runs END TO END in (LLaMA's kernels are bf16-operand only)."""
    if dtype == torch.bfloat16:
        return True
    return dtype == torch.float32 and name.lower() in LAYER_LIST_FAMILIES


def load_model(directory: str, device="cpu", dtype=torch.bfloat16):
    name, _, model_cls = resolve(directory)
    if not supports_dtype(name, dtype):
        raise ValueError(f"{name} does not run in {dtype}")
    if name == "llama":
        return model_cls.from_pretrained(directory, device=device)
    return model_cls.from_pretrained(directory, device=device, dtype=dtype)
