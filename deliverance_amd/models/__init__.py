from . import gpt2  # noqa: F401  (registers GPT2LMHeadModel)
from .causal_lm import CausalLM, load_model

__all__ = ["CausalLM", "load_model"]
