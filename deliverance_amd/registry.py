"""One registry from an architecture's name to its model.

The reference keeps a static map from ``model_type`` (upper-cased) to a (model class, config
class) pair, with ``addModel`` for extensions and ``detectModel`` on config.json
(core/src/main/java/io/teknek/deliverance/model/ModelSupport.java:54-95).  Here the key is
``architectures[0]`` of config.json, with ``model_type`` as a second name.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable, Dict, List, Sequence

from .config.specs import ConfigError, ModelConfig
from .weights.loader import TensorDecl


@dataclass(frozen=True)
class Architecture:
    """What an architecture gives the engine.

    read_config(dict)            -> ModelConfig (typed, validated; raises ConfigError)
    declare_tensors(ModelConfig) -> the checkpoint tensors it needs (names, shapes, init)
    bind_tensors(ModelConfig, tensors) -> parameters under the parts' local names:
        {"embed": {"tokens", "positions"?}, "layers": [ {"pre_mixer_norm": {...}, "mixer": {...},
          "pre_ff_norm": {...}, "feed_forward": {...}} ...], "final_norm": {...}, "head": {"weight"}}
    """
    name: str
    read_config: Callable[[dict], ModelConfig]
    declare_tensors: Callable[[ModelConfig], List[TensorDecl]]
    bind_tensors: Callable[[ModelConfig, dict], dict]
    aliases: Sequence[str] = ()
    ignore_tensors: Sequence[str] = ()
    strip_prefixes: Sequence[str] = ()


class ModelSupport:
    _by_name: Dict[str, Architecture] = {}

    @classmethod
    def add_model(cls, arch: Architecture, replace: bool = False) -> None:
        for n in (arch.name, *arch.aliases):
            key = n.lower()
            if key in cls._by_name and cls._by_name[key].name != arch.name and not replace:
                raise ValueError(f"architecture name {n!r} is already registered for {cls._by_name[key].name}")
            cls._by_name[key] = arch

    @classmethod
    def names(cls) -> List[str]:
        return sorted({a.name for a in cls._by_name.values()})

    @classmethod
    def get(cls, name: str) -> Architecture:
        a = cls._by_name.get(name.lower())
        if a is None:
            raise ConfigError(f"{name} not found in registry; known architectures: {', '.join(cls.names())}")
        return a

    @classmethod
    def detect(cls, config: dict) -> Architecture:
        """By ``architectures[0]``, else by ``model_type`` (ModelSupport.java:75-95)."""
        archs = config.get("architectures") or []
        for n in archs:
            if isinstance(n, str) and n.lower() in cls._by_name:
                return cls._by_name[n.lower()]
        mt = config.get("model_type")
        if mt is None and not archs:
            raise ConfigError("Config missing model_type field (and has no architectures).")
        if isinstance(mt, str) and mt.lower() in cls._by_name:
            return cls._by_name[mt.lower()]
        raise ConfigError(f"{archs[0] if archs else mt} not found in registry; known architectures: "
                          f"{', '.join(cls.names())}")


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.exists(path):
        raise ConfigError(f"Expecting to find config file {path}")
    with open(path) as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return d
