"""Configuration and registry (no GPU)."""
import json
import math

import pytest

import helpers
from deliverance_amd.config import ConfigError, EngineConfig, Gpt2Config
from deliverance_amd.registry import Architecture, ModelSupport, read_config_json
import deliverance_amd.models  # noqa: F401


def test_reads_its_own_keys_and_derives_sizes():
    c = Gpt2Config.from_dict(helpers.CONFIG_B)
    assert (c.n_layer, c.n_embd, c.n_head, c.vocab_size, c.n_positions) == (3, 96, 2, 1000, 96)
    assert c.head_dim == 48 and c.inner == 200
    assert c.layer_norm_epsilon == 1e-6 and c.activation_function == "gelu"
    # scale_attn_by_inverse_layer_idx: 1/sqrt(D) divided by layer + 1
    assert c.attn_scale(0) == pytest.approx(1 / math.sqrt(48))
    assert c.attn_scale(2) == pytest.approx(1 / math.sqrt(48) / 3)


def test_defaults_follow_the_architecture():
    c = Gpt2Config.from_dict(dict(n_layer=1, n_embd=32, n_head=2, vocab_size=10, n_ctx=20))
    assert c.n_positions == 20            # n_ctx is accepted where n_positions is absent
    assert c.inner == 128                 # 4 * n_embd (Gpt2Config.java:27)
    assert c.layer_norm_epsilon == 1e-5 and c.activation_function == "gelu_new"
    assert c.attn_scale(5) == pytest.approx(1 / math.sqrt(16))
    assert c.tie_word_embeddings


def test_missing_keys_are_one_error_naming_all_of_them():
    with pytest.raises(ConfigError) as e:
        Gpt2Config.from_dict(dict(n_embd=32, n_head=2))
    msg = str(e.value)
    for key in ("n_layer", "vocab_size", "n_positions"):
        assert key in msg


@pytest.mark.parametrize("patch", [dict(n_head=5), dict(n_layer=0), dict(activation_function="swish"),
                                   dict(n_inner=-3), dict(layer_norm_epsilon=0.0), dict(n_embd="64")])
def test_bad_values_are_refused(patch):
    d = dict(helpers.CONFIG_A)
    d.update(patch)
    with pytest.raises(ConfigError):
        Gpt2Config.from_dict(d)


def test_model_config_is_layers_and_a_run_order():
    mc = Gpt2Config.from_dict(helpers.CONFIG_B).to_model_config()
    assert len(mc.layers) == 3 and [c.layer for c in mc.schedule] == [0, 1, 2]
    assert [c.cache for c in mc.schedule] == [0, 1, 2] and all(c.write for c in mc.schedule)
    assert mc.n_cache_slots == 3
    scales = [l.mixer.scale for l in mc.layers]
    assert scales[0] == pytest.approx(3 * scales[2])
    assert mc.layers[1].feed_forward.inner == 200 and mc.layers[1].feed_forward.activation == "gelu"
    assert mc.layers[0].pre_mixer_norm.eps == 1e-6 and mc.final_norm.eps == 1e-6
    assert mc.embed_position.kind == "learned" and mc.embed_position.max_positions == 96
    assert mc.eos_token_ids == (999,)


def test_registry_detects_by_architecture_then_model_type():
    assert ModelSupport.detect({"architectures": ["GPT2LMHeadModel"]}).name == "GPT2LMHeadModel"
    assert ModelSupport.detect({"model_type": "gpt2"}).name == "GPT2LMHeadModel"
    assert ModelSupport.detect({"architectures": ["Unknown"], "model_type": "GPT2"}).name == "GPT2LMHeadModel"
    with pytest.raises(ConfigError, match="not found in registry"):
        ModelSupport.detect({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    with pytest.raises(ConfigError, match="missing model_type"):
        ModelSupport.detect({})


def test_registry_takes_another_architecture():
    gpt2 = ModelSupport.get("gpt2")
    toy = Architecture("ToyForTests", gpt2.read_config, gpt2.declare_tensors, gpt2.bind_tensors, aliases=("toy-test",))
    ModelSupport.add_model(toy)
    assert ModelSupport.detect({"model_type": "toy-test"}).name == "ToyForTests"
    with pytest.raises(ValueError):
        ModelSupport.add_model(Architecture("Other", gpt2.read_config, gpt2.declare_tensors, gpt2.bind_tensors,
                                            aliases=("toy-test",)))


def test_config_json_must_exist(tmp_path):
    with pytest.raises(ConfigError, match="Expecting to find config file"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text("[1, 2]")
    with pytest.raises(ConfigError):
        read_config_json(str(tmp_path))


def test_engine_config_checks():
    assert EngineConfig(dtype="bf16").dtype == "bfloat16"
    assert EngineConfig(dtype="F32").dtype == "float32"
    with pytest.raises(ValueError):
        EngineConfig(dtype="fp8")
    with pytest.raises(ValueError):
        EngineConfig(page_size=24)
    # only the page sizes that every attention kernel takes: refused here, not at the first launch
    for bad in (8, 48, 80, 128, 0, -16):
        with pytest.raises(ValueError, match="page_size must be one of"):
            EngineConfig(page_size=bad)
    assert [EngineConfig(page_size=p).page_size for p in (16, 32, 64)] == [16, 32, 64]
    assert EngineConfig().kernels == "tuned" and EngineConfig(kernels="reference").kernels == "reference"
    with pytest.raises(ValueError, match="kernels must be one of"):
        EngineConfig(kernels="fast")
