"""Large steps at the benchmark models' widths: prompts of 600 to 2,040 tokens in steps of 512 to 2,040 rows,
few layers, against the plain model, in bfloat16 and in 32-bit.

The tiny configurations never reach the products' large tiles (256 x 256, 256 x 128 and 128 x 128 with operands
straight into LDS; 128 x 128 and 128 x 64 through registers), the prefill attention's forms for long portions, or
more than a few pages a sequence; the full-depth tests reach the widths with 200 tokens.  Here a step holds a whole
prompt of 2,040 tokens, portions of 1,536 and 1,024, and portions of 512 and 576 beside decoded tokens, at widths of
768 (12 heads), 1,024 (16), 1,280 (20) and 1,600 (25), with the bounds that the tiny configurations are held to."""
import pytest

import helpers

pytestmark = [pytest.mark.gpu, pytest.mark.needs_device]

WIDTHS = {768: (12, 2), 1024: (16, 2), 1280: (20, 1), 1600: (25, 1)}      # width: heads, layers


@pytest.fixture(scope="module", params=sorted(WIDTHS))
def wide_model(request, tmp_path_factory):
    helpers.skip_in_simulation_if(True)
    width = request.param
    heads, layers = WIDTHS[width]
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", vocab_size=5003, n_positions=2048, n_layer=layers,
               n_embd=width, n_head=heads, layer_norm_epsilon=1e-5, activation_function="gelu_new", bos_token_id=0, eos_token_id=0)
    print(f"[large steps] width {width}, {heads} heads, {layers} layer(s)", flush=True)
    m = helpers.make_model(tmp_path_factory.mktemp(f"wide_{width}"), cfg, seed=width)
    yield m
    m.W = None


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_large_steps_against_the_plain_model(wide_model, dtype):
    m = wide_model
    reqs = [("a", m.prompt(2040)), ("b", m.prompt(1030, salt=1)), ("c", m.prompt(600, salt=2))]
    traces = {"a whole prompt of 2,040": (helpers.trace_whole(*reqs[0]), reqs[:1]),
              "portions of 1,536 and 504": (helpers.trace_portions(*reqs[0], sizes=(1536, 504)), reqs[:1]),
              "a portion of 1,024, then 6": (helpers.trace_portions(*reqs[1], sizes=(1024, 6)), reqs[1:2]),
              "portions of 512, 300 and 576 beside decoded tokens": (helpers.trace_mixed(reqs[1:], seed=1, max_live=2, prefill_sizes=(512, 300, 576),
                                                                                         decode_tail=4), reqs[1:])}
    for name, (steps, used) in traces.items():
        print(f"[large steps] width {m.cfg['n_embd']} {dtype}: {name}", flush=True)
        s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps), poison_freed=True)
        got = helpers.replay(s, steps)
        helpers.check_against_plain(m, got, used, dtype, f"width {m.cfg['n_embd']}, {name}")
        s.cache.manager.check()
        assert s.cache.manager.live() == []
        del s
