"""Per-request generation options, with the reference's names, meanings and defaults
(core/src/main/java/io/teknek/deliverance/generator/GeneratorParameters.java:12-28):
``temperature`` 0 is greedy; ``seed`` 42; ``ntokens`` bounds prompt + generated positions;
``max_tokens`` caps generated tokens; ``top_k`` below 1 is the legacy fraction, from 1 up a
count; ``top_p`` nucleus; ``uniform_top_p`` picks uniformly inside the nucleus; the ``xtc``
pair excludes top choices; ``log_probs``/``top_log_probs`` report the most likely tokens.
Text-level options (stop words, guided decoding, cache salt) have no meaning for an engine
that works on token ids and are not carried.

One difference is deliberate: the reference silently sets ``top_p`` to 0.10 when the
temperature is positive and no filter is given (core/.../model/AbstractGeneratorSampler.java:
107-110); here no filter means plain softmax sampling, and ``top_p=0.1`` asks for the
reference's behaviour.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Optional


@dataclass
class GeneratorParameters:
    temperature: float = 0.0
    ntokens: Optional[int] = None
    seed: Optional[int] = 42
    max_tokens: Optional[int] = None
    log_probs: bool = False
    top_log_probs: int = 0
    xtc_threshold: Optional[float] = None
    xtc_probability: Optional[float] = None
    top_k: Optional[float] = None
    top_p: Optional[float] = None
    uniform_top_p: Optional[float] = None
    ignore_eos: bool = False        # keep decoding past an end token (benchmarks)

    # builder-style setters in the reference's manner (GeneratorParameters.java:30-111)
    def with_seed(self, seed): return replace(self, seed=seed)
    def with_ntokens(self, n): return replace(self, ntokens=n)
    def with_temperature(self, t): return replace(self, temperature=float(t))
    def with_max_tokens(self, n): return replace(self, max_tokens=n)
    def with_log_probs(self, b): return replace(self, log_probs=bool(b))
    def with_top_log_probs(self, n): return replace(self, top_log_probs=int(n))
    def with_xtc_threshold(self, t): return replace(self, xtc_threshold=float(t))
    def with_xtc_probability(self, p): return replace(self, xtc_probability=float(p))
    def with_top_k(self, k): return replace(self, top_k=float(k))
    def with_top_p(self, p): return replace(self, top_p=float(p))
    def with_uniform_top_p(self, p): return replace(self, uniform_top_p=float(p))

    def validate(self) -> None:
        """The argument checks of AbstractGeneratorSampler.java:161-176,268-279."""
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if self.top_k is not None and self.top_k <= 0:
            raise ValueError("topK must be > 0")
        if self.top_p is not None and not (0.0 < self.top_p <= 1.0):
            raise ValueError("topP must be in (0, 1]")
        if self.uniform_top_p is not None and not (0.0 < self.uniform_top_p <= 1.0):
            raise ValueError("uniformTopP must be in (0, 1]")
        if self.uniform_top_p is not None and self.top_p is None:
            raise ValueError("uniformTopP requires topP")
        if self.uniform_top_p is not None and self.temperature == 0:
            raise ValueError("uniformTopP requires temperature > 0")
        if self.top_k is not None and self.xtc_threshold is not None and self.temperature > 0:
            raise ValueError("can not enable topk and xtc")
        if self.max_tokens is not None and self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        if self.top_log_probs < 0:
            raise ValueError("top_log_probs must be >= 0")
