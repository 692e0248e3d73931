"""The random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed, through the same registry and tensor declarations as loading."""
from __future__ import annotations

import torch

from .registry import ModelSupport
from .weights.loader import write_random_model


def random_model(folder: str, config: dict, seed: int, dtype: torch.dtype = torch.bfloat16) -> str:
    """``config`` holds the architecture's own config.json keys (with ``architectures`` or
    ``model_type``).  Returns ``folder``."""
    from . import models  # noqa: F401  (registers the architectures)
    arch = ModelSupport.detect(config)
    mc = arch.read_config(config)
    out_cfg = dict(mc.raw) if mc.raw else dict(config)
    for k, v in config.items():
        out_cfg.setdefault(k, v)
    return write_random_model(folder, out_cfg, arch.declare_tensors(mc), seed, dtype)
