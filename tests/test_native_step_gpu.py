"""The layer loop issued from C++ in one call (``da_run_step``) against the same step run part by part:
the same kernels with the same arguments, so the logits must agree bit for bit, in every way of cutting
and through the recorded decode steps; and the plan is only made for what it describes."""
import numpy as np
import pytest

import helpers

pytestmark = [pytest.mark.gpu, pytest.mark.needs_device]


def both_ways(model, steps, max_tokens, **options):
    runs = []
    for native in (True, False):
        s = helpers.trace_session(model.folder, "bfloat16", max_tokens, poison_freed=True, native_step=native, **options)
        assert (s.runner.native is not None) == native
        runs.append(helpers.replay(s, steps))
        s.cache.manager.check()
    return runs


@pytest.mark.parametrize("name", ["A", "B", "B32"])
def test_native_step_gives_the_bits_of_the_parts(models, name):
    m = models[name]
    reqs = [(f"r{i}", m.prompt(n, salt=80 + i)) for i, n in enumerate((40, 17, 56, 5, 33, 64, 23))]
    for steps in (helpers.trace_mixed(reqs, seed=4), helpers.trace_whole(*reqs[2]), helpers.trace_bulk_then_single(*reqs[5], 32),
                  helpers.trace_portions(*reqs[0], (7, 2, 13, 1))):
        native, parts = both_ways(m, steps, max(helpers.max_live_tokens(steps), 128))
        assert native.keys() == parts.keys()
        for rid in native:
            assert np.array_equal(native[rid], parts[rid]), rid
    helpers.check_against_plain(m, native, [reqs[0]], "bfloat16", "native step")


def test_native_step_inside_recorded_decode_steps(models):
    from test_engine_paths_gpu import decode_trace
    m = models["B"]
    reqs = [(f"g{i}", m.prompt(n, salt=90 + i)) for i, n in enumerate((32, 17, 64, 33, 9))]
    steps = decode_trace(reqs, [3, 5, 9, 14, 6])
    native, parts = both_ways(m, steps, 512, use_graphs=True, sample=True)
    for rid in native:
        assert np.array_equal(native[rid], parts[rid]), rid
    helpers.check_against_plain(m, native, reqs, "bfloat16", "native step, graphs")


def test_native_step_at_a_width_with_separate_norms_and_split_decode_attention(tmp_path):
    """A width of 1,600 (the norm is a kernel of its own beyond a few rows) and a context of 2,200 tokens
    (decode attention shares the keys out): the branches of the C++ loop that the tiny models do not reach."""
    from test_engine_paths_gpu import decode_trace
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=1600, n_head=25, vocab_size=301,
               n_positions=2304, layer_norm_epsilon=1e-5, activation_function="gelu_new", bos_token_id=0, eos_token_id=1)
    m = helpers.make_model(tmp_path, cfg, seed=21)
    reqs = [("far", m.prompt(2200, salt=1)), ("near", m.prompt(300, salt=2))]
    steps = decode_trace(reqs, [6, 6])
    native, parts = both_ways(m, steps, 4096)
    for rid in native:
        assert np.array_equal(native[rid], parts[rid]), rid


def test_the_plan_is_made_only_for_what_it_describes(models):
    m = models["A"]
    assert helpers.trace_session(m.folder, "float32", 128).runner.native is None
    assert helpers.trace_session(m.folder, "bfloat16", 128, kernels="reference").runner.native is None
    s = helpers.trace_session(m.folder, "bfloat16", 128)
    assert s.runner.native is not None
    # with a debug hook the parts run one by one (the hook looks between the kernels)
    seen = []
    s.runner.debug_hook = lambda layer, stage, t: seen.append(stage)
    helpers.replay(s, helpers.trace_whole("d", m.prompt(9)))
    assert "attention_value" in seen
