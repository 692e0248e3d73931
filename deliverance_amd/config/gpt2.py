"""Typed GPT-2 configuration, read from the architecture's own config.json keys.

The reference reads ``n_ctx, n_embd, n_head, n_layer, layer_norm_epsilon, vocab_size,
bos_token_id, eos_token_id`` and fixes the MLP width at ``4 * n_embd`` and the activation
at erf-GELU (core/src/main/java/io/teknek/deliverance/model/gpt2/Gpt2Config.java:13-39).
This class also honours ``n_positions`` (preferred over ``n_ctx``), ``n_inner``,
``activation_function``, ``scale_attn_by_inverse_layer_idx`` and ``tie_word_embeddings``,
and treats a missing required key as an error instead of a silent zero
(the reference's mapper tolerates missing keys: core/.../JsonUtils.java:15-19).
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

from .specs import (AttentionSpec, ConfigError, DenseFeedForwardSpec, LayerCall, LayerSpec,
                    ModelConfig, NormSpec, PositionSpec)

KNOWN_ACTIVATIONS = ("gelu_new", "gelu", "gelu_pytorch_tanh", "relu", "silu")


@dataclass(frozen=True)
class Gpt2Config:
    n_layer: int
    n_embd: int
    n_head: int
    vocab_size: int
    n_positions: int
    n_inner: Optional[int] = None
    layer_norm_epsilon: float = 1e-5
    activation_function: str = "gelu_new"
    scale_attn_by_inverse_layer_idx: bool = False
    tie_word_embeddings: bool = True
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None

    ARCHITECTURE = "GPT2LMHeadModel"
    MODEL_TYPE = "gpt2"
    REQUIRED = ("n_layer", "n_embd", "n_head", "vocab_size")

    # ---- reading -----------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "Gpt2Config":
        missing = [k for k in cls.REQUIRED if d.get(k) is None]
        if d.get("n_positions") is None and d.get("n_ctx") is None:
            missing.append("n_positions (or n_ctx)")
        if missing:
            raise ConfigError("GPT-2 config.json lacks required keys: " + ", ".join(missing))

        def _int(key, value):
            if isinstance(value, bool) or not isinstance(value, int):
                raise ConfigError(f"config key {key!r} must be an integer, found {value!r}")
            return value

        n_positions = d.get("n_positions") if d.get("n_positions") is not None else d["n_ctx"]
        n_inner = d.get("n_inner")
        cfg = cls(
            n_layer=_int("n_layer", d["n_layer"]),
            n_embd=_int("n_embd", d["n_embd"]),
            n_head=_int("n_head", d["n_head"]),
            vocab_size=_int("vocab_size", d["vocab_size"]),
            n_positions=_int("n_positions", n_positions),
            n_inner=None if n_inner is None else _int("n_inner", n_inner),
            layer_norm_epsilon=float(d.get("layer_norm_epsilon", 1e-5)),
            activation_function=str(d.get("activation_function", "gelu_new")),
            scale_attn_by_inverse_layer_idx=bool(d.get("scale_attn_by_inverse_layer_idx", False)),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", True)),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=d.get("eos_token_id"),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for key in ("n_layer", "n_embd", "n_head", "vocab_size", "n_positions"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config key {key!r} must be positive, found {getattr(self, key)}")
        if self.n_inner is not None and self.n_inner <= 0:
            raise ConfigError(f"config key 'n_inner' must be positive, found {self.n_inner}")
        if self.n_embd % self.n_head != 0:
            raise ConfigError(
                f"n_embd ({self.n_embd}) is not a multiple of n_head ({self.n_head})")
        if self.activation_function not in KNOWN_ACTIVATIONS:
            raise ConfigError(
                f"activation_function {self.activation_function!r} is not one of {KNOWN_ACTIVATIONS}")
        if not (self.layer_norm_epsilon > 0.0):
            raise ConfigError(f"layer_norm_epsilon must be > 0, found {self.layer_norm_epsilon}")

    # ---- derived sizes -----------------------------------------------------------
    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    @property
    def inner(self) -> int:
        return self.n_inner if self.n_inner is not None else 4 * self.n_embd

    def attn_scale(self, layer: int) -> float:
        """1/sqrt(D) (core/.../generator/CausalSelfAttention.java:203), divided by
        ``layer + 1`` when ``scale_attn_by_inverse_layer_idx`` is set."""
        s = 1.0 / math.sqrt(self.head_dim)
        if self.scale_attn_by_inverse_layer_idx:
            s /= float(layer + 1)
        return s

    def to_dict(self) -> dict:
        d = {
            "architectures": [self.ARCHITECTURE],
            "model_type": self.MODEL_TYPE,
            "n_layer": self.n_layer,
            "n_embd": self.n_embd,
            "n_head": self.n_head,
            "n_inner": self.n_inner,
            "vocab_size": self.vocab_size,
            "n_positions": self.n_positions,
            "n_ctx": self.n_positions,
            "layer_norm_epsilon": self.layer_norm_epsilon,
            "activation_function": self.activation_function,
            "scale_attn_by_inverse_layer_idx": self.scale_attn_by_inverse_layer_idx,
            "tie_word_embeddings": self.tie_word_embeddings,
        }
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d

    # ---- the model as parts ------------------------------------------------------
    def to_model_config(self) -> ModelConfig:
        """Pre-LayerNorm blocks (core/.../generator/TransformerBlock.java:35-41,169-198),
        learned absolute positions added to the token embedding
        (core/.../model/gpt2/Gpt2Model.java:42-48), head tied to ``wte``
        (Gpt2Model.java:54-71)."""
        norm = NormSpec("layernorm", self.n_embd, self.layer_norm_epsilon, bias=True)
        layers = []
        for l in range(self.n_layer):
            mixer = AttentionSpec(
                kind="attention", width=self.n_embd, n_heads=self.n_head, n_kv_heads=self.n_head,
                head_dim=self.head_dim, scale=self.attn_scale(l), qkv_bias=True, out_bias=True,
                window=None, position=None)
            ff = DenseFeedForwardSpec(kind="dense", width=self.n_embd, inner=self.inner,
                                      activation=self.activation_function, bias=True)
            layers.append(LayerSpec(mixer=mixer, feed_forward=ff, pre_mixer_norm=norm,
                                    pre_ff_norm=norm, weight_prefix=f"h.{l}."))
        schedule: Tuple[LayerCall, ...] = tuple(LayerCall(l, l, True) for l in range(self.n_layer))
        eos = () if self.eos_token_id is None else (int(self.eos_token_id),)
        return ModelConfig(
            architecture=self.ARCHITECTURE,
            vocab_size=self.vocab_size,
            width=self.n_embd,
            max_positions=self.n_positions,
            layers=tuple(layers),
            schedule=schedule,
            embed_position=PositionSpec("learned", self.n_positions),
            final_norm=norm,
            tie_word_embeddings=self.tie_word_embeddings,
            bos_token_id=self.bos_token_id,
            eos_token_ids=eos,
            raw=self.to_dict(),
        )
