"""Typed descriptions of the parts a model is assembled from.

A model configuration (see ``gpt2.py``) turns the keys of its ``config.json`` into these
records: one :class:`LayerSpec` per layer and a run order (:class:`LayerCall` list).  The
parts in ``deliverance_amd.parts`` are built from the records alone, so a part never
learns which model it sits in, and two layers of one model may carry different mixers
and feed-forwards.

The reference keeps the same facts as fields of one flat ``Config`` object
(safetensors/src/main/java/io/teknek/deliverance/safetensors/Config.java:315-377) and as
constructor arguments of its block classes
(core/src/main/java/io/teknek/deliverance/generator/TransformerBlock.java:26-41).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a model (missing key, bad value)."""


@dataclass(frozen=True)
class NormSpec:
    kind: str            # "layernorm" (others are added through parts.register_norm)
    width: int
    eps: float
    bias: bool = True


@dataclass(frozen=True)
class PositionSpec:
    """Where a token's position enters the model.

    ``kind == "learned"``: a table of ``max_positions`` rows is added to the token
    embedding.  ``kind == "none"``: nothing.  Other kinds may act on queries and keys
    inside an attention mixer (see ``parts.positions``).
    """
    kind: str
    max_positions: int = 0
    params: Tuple[Tuple[str, float], ...] = ()


@dataclass(frozen=True)
class AttentionSpec:
    kind: str            # "attention"
    width: int           # model width E
    n_heads: int
    n_kv_heads: int
    head_dim: int
    scale: float         # multiplies q.k before the softmax
    qkv_bias: bool = True
    out_bias: bool = True
    window: Optional[int] = None     # None: every earlier key; w: the last w keys
    position: Optional[PositionSpec] = None  # acts on q and k (none for learned tables)


@dataclass(frozen=True)
class DenseFeedForwardSpec:
    kind: str            # "dense"
    width: int
    inner: int
    activation: str      # "gelu_new" | "gelu" | "gelu_pytorch_tanh" | "relu" | "silu"
    bias: bool = True


@dataclass(frozen=True)
class LayerSpec:
    """One block: ``x += mixer(norm1(x)); x += ff(norm2(x))`` with optional norm slots.

    The reference's block has five optional norm places
    (core/.../generator/TransformerBlock.java:26-32); the pre-norm pair is what its
    GPT-2 uses (TransformerBlock.java:35-41).  ``post_block_norm`` is the fifth (applied to
    the stream when both parts have joined it, TransformerBlock.java:199);
    ``residual_multiplier`` scales a part's output (after the norm behind it, if any) before
    it joins the stream (TransformerBlock.java:260-272; 1: plain addition).
    """
    mixer: object
    feed_forward: object
    pre_mixer_norm: Optional[NormSpec] = None
    post_mixer_norm: Optional[NormSpec] = None
    pre_ff_norm: Optional[NormSpec] = None
    post_ff_norm: Optional[NormSpec] = None
    weight_prefix: str = ""
    post_block_norm: Optional[NormSpec] = None
    residual_multiplier: float = 1.0


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``ModelConfig.layers`` (a layer may be named twice), ``cache`` is
    the cache slot its mixer uses, and ``write`` is False when the mixer only reads a
    slot that another call has filled in the same step.
    """
    layer: int
    cache: int
    write: bool = True


@dataclass(frozen=True)
class ModelConfig:
    """What every architecture's typed configuration provides to the engine."""
    architecture: str
    vocab_size: int
    width: int
    max_positions: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[LayerCall, ...]
    embed_position: PositionSpec
    final_norm: Optional[NormSpec]
    tie_word_embeddings: bool
    bos_token_id: Optional[int]
    eos_token_ids: Tuple[int, ...]
    raw: dict = field(default_factory=dict, compare=False, hash=False)
    embed_scale: float = 1.0        # multiplies the token embedding before positions are added
    # logits are divided by it (the reference's logitMultiplier, AbstractGeneratorSampler.java:117-120)
    logit_multiplier: float = 1.0

    @property
    def n_cache_slots(self) -> int:
        return 1 + max((c.cache for c in self.schedule), default=-1)
