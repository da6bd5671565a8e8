"""Model registry: which class serves a config, and how a model directory is read.

A directory's ``config.json`` either carries ``architecture`` (a layer-list design: the config
lists its layers, models/hybrid.py) or the Hugging Face keys (``model_type``: llama / mistral /
mixtral / gpt2, models/checkpoint.py)."""
from __future__ import annotations

import json
from pathlib import Path
from typing import Optional, Union

import torch

from .checkpoint import SafetensorsDir, config_from_hf, load_checkpoint
from .config import DESIGN_TRAITS, HybridConfig, ModelConfig, hybrid_config_from_dict
from .hybrid import HybridLM
from .llama import CausalLM

# config.arch -> model class
MODEL_CLASSES = {"llama": CausalLM, "gpt2": CausalLM, "dunesun": HybridLM, "kisutar": HybridLM, "bitonex": HybridLM,
                 "levovik": HybridLM}
# layer-list designs by the ``architecture`` value of their config.json (lower case)
LAYER_LIST_ARCHS = set(DESIGN_TRAITS)


def config_from_dir(path: Union[str, Path], name: Optional[str] = None):
    """The model config of a directory holding ``config.json`` (either dialect)."""
    p = Path(path)
    if p.is_dir():
        p = p / "config.json"
    c = json.loads(p.read_text())
    arch = str(c.get("architecture", "")).lower()
    if arch:
        if arch not in LAYER_LIST_ARCHS:
            raise ValueError(f"unknown architecture {c['architecture']!r} (known: {sorted(LAYER_LIST_ARCHS)})")
        return hybrid_config_from_dict(c, name or p.parent.name)
    return config_from_hf(c, name or p.parent.name)


def build_model(cfg, device="cpu", dtype=torch.bfloat16, seed: int = 0, pstate=None, weights: Optional[str] = None):
    """Instantiate ``cfg``'s model class; ``weights``: a model directory to load."""
    cls = MODEL_CLASSES.get(cfg.arch)
    if cls is None:
        raise KeyError(f"no model class for arch {cfg.arch!r} (known: {sorted(MODEL_CLASSES)})")
    if isinstance(cfg, HybridConfig):
        src = SafetensorsDir(weights) if weights else None
        return cls(cfg, device=device, dtype=dtype, seed=seed, pstate=pstate, weights=src)
    assert isinstance(cfg, ModelConfig)
    model = cls(cfg, device=device, dtype=dtype, seed=seed, pstate=pstate, init="empty" if weights else "random")
    if weights:
        load_checkpoint(model, weights)
    return model
