"""deliverance_amd: a small, whole inference engine for one GPU (MI355X, gfx950).

    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    model = AutoModelForCausalLM.from_pretrained(folder, dtype="bfloat16")
    out = model.generate([1, 2, 3], GeneratorParameters().with_max_tokens(16))
"""
from .config import EngineConfig, Gpt2Config
from .registry import Architecture, ModelSupport
from .sampling import GeneratorParameters

__version__ = "0.1.0"


def __getattr__(name):
    # The engine pulls in torch and the kernel library; configuration, weights, cache manager
    # and scheduler stay importable without them.
    if name in ("AutoModelForCausalLM", "CausalLanguageModel", "Response"):
        from .engine import engine as _e
        return getattr(_e, name)
    if name == "random_model":
        from .random_model import random_model
        return random_model
    raise AttributeError(name)


__all__ = ["AutoModelForCausalLM", "CausalLanguageModel", "Response", "GeneratorParameters", "EngineConfig",
           "Gpt2Config", "ModelSupport", "Architecture", "random_model"]
