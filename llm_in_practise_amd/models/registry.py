"""Which model class a checkpoint folder needs, from its ``config.json``.

``architecture`` / ``architectures`` / ``model_type`` name the design; every entry maps to a loader with the same
call (``from_pretrained(path, dtype=, device=)``) that returns a causal LM the serving engine can drive
(``.model``, ``.lm_head``, ``.config``; models with per-sequence state beyond K/V also ``.make_cache``).
"""
from __future__ import annotations

import json
import os


def _qwen():
    from .qwen3 import Qwen3ForCausalLM
    return Qwen3ForCausalLM


def _mobupel():
    from .mobupel import MobupelForCausalLM
    return MobupelForCausalLM


def _dogudra():
    from .dogudra import DogudraForCausalLM
    return DogudraForCausalLM


def _kitonex():
    from .kitonex import KitonexForCausalLM
    return KitonexForCausalLM


def _mamivik():
    from .mamivik import MamivikForCausalLM
    return MamivikForCausalLM


REGISTRY = {
    "qwen3": _qwen, "qwen2": _qwen, "qwen3forcausallm": _qwen, "qwen2forcausallm": _qwen,
    "mobupel": _mobupel, "mobupelforcausallm": _mobupel,
    "dogudra": _dogudra, "dogudraforcausallm": _dogudra,
    "kitonex": _kitonex, "kitonexforcausallm": _kitonex,
    "mamivik": _mamivik, "mamivikforcausallm": _mamivik,
}


def architecture_of(config: dict) -> str:
    names = [config.get("architecture"), config.get("model_type")] + list(config.get("architectures") or [])
    for n in names:
        if isinstance(n, str) and n.lower() in REGISTRY:
            return n.lower()
    raise ValueError(f"no model class for architecture {[n for n in names if n]} (known: {sorted(REGISTRY)})")


def model_class(path_or_config):
    cfg = path_or_config
    if not isinstance(cfg, dict):
        with open(os.path.join(path_or_config, "config.json")) as f:
            cfg = json.load(f)
    return REGISTRY[architecture_of(cfg)]()


def load_causal_lm(path: str, dtype=None, device=None, **kw):
    import torch
    return model_class(path).from_pretrained(path, dtype=dtype or torch.bfloat16, device=device, **kw)
