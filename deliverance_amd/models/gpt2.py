"""GPT-2: which checkpoint tensors feed which part.

Names and load-time transforms follow core/src/main/java/io/teknek/deliverance/model/gpt2/
Gpt2Model.java:36-119: ``wte``/``wpe`` embeddings; per layer ``h.{i}.attn.c_attn`` and
``c_proj``, ``h.{i}.mlp.c_fc`` and ``c_proj`` stored [in, out] and transposed at load
(:81-82,93,103,105); ``ln_1``/``ln_2``; ``ln_f`` and ``wte`` again for the head (:54-71).
The fused q|k|v projection stays one matrix here instead of being split in three.
"""
from __future__ import annotations

from typing import List

from ..config.gpt2 import Gpt2Config
from ..config.specs import ModelConfig
from ..registry import Architecture, ModelSupport
from ..weights.loader import TensorDecl

# Random-weights distributions: weights and biases N(0, 0.02), norm gains 1 + N(0, 0.1),
# norm biases N(0, 0.02), position table N(0, 0.01).
W_STD, GAIN_STD, POS_STD = 0.02, 0.1, 0.01


def read_config(d: dict) -> ModelConfig:
    return Gpt2Config.from_dict(d).to_model_config()


def declare_tensors(mc: ModelConfig) -> List[TensorDecl]:
    E, V, P = mc.width, mc.vocab_size, mc.max_positions
    out = [TensorDecl("wte.weight", (V, E), "normal", W_STD),
           TensorDecl("wpe.weight", (P, E), "normal", POS_STD)]
    for spec in mc.layers:
        p = spec.weight_prefix
        a, f = spec.mixer, spec.feed_forward
        qkv = (a.n_heads + 2 * a.n_kv_heads) * a.head_dim
        out += [
            TensorDecl(p + "ln_1.weight", (E,), "ones_plus_normal", GAIN_STD),
            TensorDecl(p + "ln_1.bias", (E,), "normal", W_STD),
            TensorDecl(p + "attn.c_attn.weight", (E, qkv), "normal", W_STD),
            TensorDecl(p + "attn.c_attn.bias", (qkv,), "normal", W_STD),
            TensorDecl(p + "attn.c_proj.weight", (a.n_heads * a.head_dim, E), "normal", W_STD),
            TensorDecl(p + "attn.c_proj.bias", (E,), "normal", W_STD),
            TensorDecl(p + "ln_2.weight", (E,), "ones_plus_normal", GAIN_STD),
            TensorDecl(p + "ln_2.bias", (E,), "normal", W_STD),
            TensorDecl(p + "mlp.c_fc.weight", (E, f.inner), "normal", W_STD),
            TensorDecl(p + "mlp.c_fc.bias", (f.inner,), "normal", W_STD),
            TensorDecl(p + "mlp.c_proj.weight", (f.inner, E), "normal", W_STD),
            TensorDecl(p + "mlp.c_proj.bias", (E,), "normal", W_STD),
        ]
    out += [TensorDecl("ln_f.weight", (E,), "ones_plus_normal", GAIN_STD),
            TensorDecl("ln_f.bias", (E,), "normal", W_STD)]
    if not mc.tie_word_embeddings:
        out.append(TensorDecl("lm_head.weight", (V, E), "normal", W_STD))
    return out


def bind_tensors(mc: ModelConfig, t: dict) -> dict:
    layers = []
    for spec in mc.layers:
        p = spec.weight_prefix
        layers.append({
            "pre_mixer_norm": {"weight": t[p + "ln_1.weight"], "bias": t[p + "ln_1.bias"]},
            "mixer": {"qkv_weight": t[p + "attn.c_attn.weight"].t(), "qkv_bias": t[p + "attn.c_attn.bias"],
                      "out_weight": t[p + "attn.c_proj.weight"].t(), "out_bias": t[p + "attn.c_proj.bias"]},
            "pre_ff_norm": {"weight": t[p + "ln_2.weight"], "bias": t[p + "ln_2.bias"]},
            "feed_forward": {"fc_weight": t[p + "mlp.c_fc.weight"].t(), "fc_bias": t[p + "mlp.c_fc.bias"],
                             "proj_weight": t[p + "mlp.c_proj.weight"].t(), "proj_bias": t[p + "mlp.c_proj.bias"]},
        })
    head = t["wte.weight"] if mc.tie_word_embeddings else t["lm_head.weight"]
    return {
        "embed": {"tokens": t["wte.weight"], "positions": {"table": t["wpe.weight"]}},
        "layers": layers,
        "final_norm": {"weight": t["ln_f.weight"], "bias": t["ln_f.bias"]},
        "head": {"weight": head},
    }


GPT2 = Architecture(
    name=Gpt2Config.ARCHITECTURE,
    read_config=read_config,
    declare_tensors=declare_tensors,
    bind_tensors=bind_tensors,
    aliases=(Gpt2Config.MODEL_TYPE,),
    # buffers some checkpoints carry and the model never reads; a tied model may also store its head
    ignore_tensors=("h.*.attn.bias", "h.*.attn.masked_bias", "lm_head.weight"),
    strip_prefixes=("transformer.",),
)
ModelSupport.add_model(GPT2)
