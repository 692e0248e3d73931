"""Configurations drawn at random (head sizes 16 to 256 in steps of 16, one to seven heads, inner
widths that are no multiple of 8, odd vocabularies, every page size, every activation) replayed
mixed, with pages used again, and whole, against the plain implementation, in 32-bit and in
bfloat16: a size that a kernel does not take must be refused or served by another kernel, never
answered wrongly.

Seeds 5 and 11 hold products whose inner size is 32, below one 64-wide slab of the block-tile
kernel: its loads past K once fell back to an address that was itself past K (the thread's own
chunk of the first slab, not the row's first chunk) and read up to 64 bytes behind the last row of
an operand, which faults only when the operand ends where mapped memory ends.  tests/test_simt.py
runs these two seeds on the CPU with every operand between protected pages."""
import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = np.random.default_rng(seed)
    D = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 256]))
    H = int(rng.integers(1, 8)) if D <= 128 else int(rng.integers(1, 3))
    inner = [None, int(rng.integers(3, 60)) * 8, int(rng.integers(17, 400))][int(rng.integers(0, 3))]
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=int(rng.integers(1, 4)), n_embd=D * H,
               n_head=H, vocab_size=int(rng.integers(130, 3000)), n_positions=int(rng.choice([96, 160, 333, 520])),
               layer_norm_epsilon=float(rng.choice([1e-5, 1e-6, 1e-3])),
               activation_function=str(rng.choice(["gelu_new", "gelu", "gelu_pytorch_tanh"])),
               scale_attn_by_inverse_layer_idx=bool(rng.integers(0, 2)), bos_token_id=0, eos_token_id=1)
    if inner is not None:
        cfg["n_inner"] = inner
    return cfg, int(rng.choice([16, 32, 64])), rng


# seeds chosen so that the head sizes 16, 32, 80, 96, 112, 128, 160 and 256 all occur
@pytest.mark.parametrize("seed", [1, 4, 5, 7, 11, 13, 212, 218])
def test_random_configuration_mixed_and_whole(tmp_path, seed):
    cfg, page, rng = draw_config(seed)
    m = helpers.make_model(tmp_path, cfg, seed)
    P = cfg["n_positions"]
    lengths = [int(x) for x in rng.integers(1, P - 1, size=4)] + [P - 1]
    reqs = [(f"r{i}", m.prompt(n, salt=i)) for i, n in enumerate(lengths)]
    steps = helpers.trace_mixed(reqs, seed=seed, prefill_sizes=(9, 2, 67, 4, 130, 33), decode_tail=int(rng.integers(1, 20)))
    unit = max(64, page)
    for dtype in ("float32", "bfloat16"):
        s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps, round_to=unit), page)
        got = helpers.replay(s, steps)
        helpers.check_against_plain(m, got, reqs, dtype, f"mixed {cfg} page {page}")
        s.cache.manager.check()
        assert s.cache.manager.pools[0].n_free == s.cache.n_pages
        s = helpers.trace_session(m.folder, dtype, -(-P // unit) * unit, page)
        got = helpers.replay(s, helpers.trace_whole(*reqs[-1]))
        helpers.check_against_plain(m, got, reqs[-1:], dtype, f"whole {cfg} page {page}")


# (width, heads): head sizes 10, 24, 25 and 40; a width of 100 is no multiple of 8 either, so its products
# leave the matrix cores as well
@pytest.mark.parametrize("width,heads", [(40, 4), helpers.quick(72, 3), (100, 4), (120, 3)])
def test_head_sizes_that_are_no_multiple_of_16(tmp_path, width, heads):
    """config.json allows any n_embd / n_head: the 32-bit path takes every head size up to 256, and
    bfloat16 serves those that the matrix-core attention kernels do not take through the plain
    attention kernel (the reference divides likewise and asks nothing more of the head size:
    safetensors/src/main/java/io/teknek/deliverance/safetensors/Config.java:340-354)."""
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=width, n_head=heads,
               vocab_size=211, n_positions=96, layer_norm_epsilon=1e-5, activation_function="gelu_new",
               bos_token_id=0, eos_token_id=1)
    m = helpers.make_model(tmp_path, cfg, seed=width)
    reqs = [(f"r{i}", m.prompt(n, salt=i)) for i, n in enumerate((70, 9, 33, 95))]
    steps = helpers.trace_mixed(reqs, seed=width, prefill_sizes=(9, 2, 40, 4), decode_tail=7)
    for dtype in ("float32", "bfloat16"):
        s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps), poison_freed=True)
        got = helpers.replay(s, steps)
        helpers.check_against_plain(m, got, reqs, dtype, f"head size {width // heads}, mixed")
        got = helpers.replay(s, helpers.trace_bulk_then_single(*reqs[3], 32))
        helpers.check_against_plain(m, got, reqs[3:], dtype, f"head size {width // heads}, bulk+single")
        s.cache.manager.check()


def test_head_sizes_beyond_the_kernels_are_refused(tmp_path):
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=1, n_embd=272, n_head=1,
               vocab_size=50, n_positions=32)
    m = helpers.make_model(tmp_path, cfg, seed=1)
    with pytest.raises(ValueError, match="head size 272"):
        helpers.trace_session(m.folder, "float32", 64)
