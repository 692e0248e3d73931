from .specs import (AttentionSpec, ConfigError, DenseFeedForwardSpec, LayerCall, LayerSpec,
                    ModelConfig, NormSpec, PositionSpec)
from .gpt2 import Gpt2Config
from .engine_config import EngineConfig

__all__ = ["AttentionSpec", "ConfigError", "DenseFeedForwardSpec", "LayerCall", "LayerSpec",
           "ModelConfig", "NormSpec", "PositionSpec", "Gpt2Config", "EngineConfig"]
