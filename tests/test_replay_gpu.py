"""Trace replay against the plain implementation, in 32-bit and in bfloat16: each request
alone and whole; most of it in one step and the last 32 tokens one by one; in portions of
changing size; and mixed, with so few pages that they are used again."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
LENGTHS = {"A": (5, 17, 40, 56), "B": (1, 9, 33, 64, 88)}


def session_for(model, dtype, max_tokens, page_size=16):
    return helpers.trace_session(model.folder, dtype, max_tokens, page_size, poison_freed=True)   # pages that go back are NaN again


def requests_of(model, name):
    return [(f"{name}{n}", model.prompt(n)) for n in LENGTHS[name[0]]]


# A, B: stored in bfloat16; A32, B32: stored in 32-bit (B32 with a head of its own)
NAMES = ["A", "B", "A32", "B32"]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole(models, name, dtype):
    m = models[name]
    reqs = requests_of(m, name)
    s = session_for(m, dtype, 128)
    for rid, ids in reqs:
        got = helpers.replay(s, helpers.trace_whole(rid, ids))
        helpers.check_against_plain(m, got, [(rid, ids)], dtype, "whole")
    s.cache.manager.check()
    assert s.cache.manager.pools[0].n_free == s.cache.n_pages


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_bulk_then_last_32_one_by_one(models, name, dtype):
    m = models[name]
    s = session_for(m, dtype, 128)
    for rid, ids in requests_of(m, name)[2:]:
        got = helpers.replay(s, helpers.trace_bulk_then_single(rid, ids, 32))
        helpers.check_against_plain(m, got, [(rid, ids)], dtype, "bulk+single")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(models, name, dtype):
    m = models[name]
    s = session_for(m, dtype, 128)
    for sizes in ((7, 2, 13, 3, 5, 2), (7,), (2,), (16, 1, 15, 17)):
        for rid, ids in requests_of(m, name)[1:]:
            got = helpers.replay(s, helpers.trace_portions(rid, ids, sizes))
            helpers.check_against_plain(m, got, [(rid, ids)], dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_with_pages_used_again(models, name, dtype):
    m = models[name]
    lengths = {"A": (40, 17, 56, 5, 33, 64, 23, 48), "B": (64, 9, 33, 88, 1, 50, 17, 40)}[name[0]]
    reqs = [(f"r{i}", m.prompt(n, salt=i)) for i, n in enumerate(lengths)]
    steps = helpers.trace_mixed(reqs, seed=3)
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len({len(e["tokens"]) == 1 for e in s["entries"]}) == 2 for s in steps)   # portions beside single tokens
    budget = helpers.max_live_tokens(steps)
    s = session_for(m, dtype, budget)
    assert sum(-(-n // 16) for n in lengths) > s.cache.n_pages        # the pool cannot hold all: pages come back
    got = helpers.replay(s, steps)
    helpers.check_against_plain(m, got, reqs, dtype, "mixed")
    s.cache.manager.check()
    assert s.cache.manager.pools[0].n_free == s.cache.n_pages


@pytest.mark.parametrize("dtype", DTYPES)
def test_cutting_does_not_change_logits_beyond_rounding(model_b, dtype):
    """The same request four ways; the engine against itself, tighter than against the plain model."""
    m = model_b
    ids = m.prompt(88)
    runs = []
    for steps in (helpers.trace_whole("x", ids), helpers.trace_bulk_then_single("x", ids, 32),
                  helpers.trace_portions("x", ids), helpers.trace_portions("x", ids, (2,))):
        s = session_for(m, dtype, 128)
        runs.append(helpers.replay(s, steps)["x"])
    tol = 1e-6 if dtype == "float32" else 6e-3
    for r in runs[1:]:
        assert np.abs(r - runs[0]).max() <= tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_neighbours_do_not_change_logits_beyond_rounding(model_b, dtype):
    """A request alone and the same request beside three others (portions beside decoded tokens, longer and
    shorter neighbours, which change the attention kernels' forms and the products' row counts): 32-bit sums
    keep their order whatever shares the step; in bfloat16 the forms that a step takes depend on its shape,
    so a request's rounding may differ with its neighbours, within the bound that cutting is held to."""
    m = model_b
    ids = m.prompt(88, salt=7)
    alone = helpers.replay(session_for(m, dtype, 128), helpers.trace_bulk_then_single("x", ids, 24))["x"]
    others = [("n%d" % i, m.prompt(n, salt=20 + i)) for i, n in enumerate((96, 33, 64))]
    steps = helpers.trace_mixed([("x", ids)] + others, seed=3, max_live=4)
    s = session_for(m, dtype, helpers.max_live_tokens(steps))
    beside = helpers.replay(s, steps)["x"]
    assert beside.shape == alone.shape
    tol = 1e-6 if dtype == "float32" else 6e-3
    assert np.abs(beside - alone).max() <= tol


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_first_tokens(model_a, dtype):
    m = model_a
    ids = m.prompt(128)                       # the whole context, one token a step from the first
    s = session_for(m, dtype, 128)
    got = helpers.replay(s, helpers.trace_bulk_then_single("d", ids, 127))
    helpers.check_against_plain(m, got, [("d", ids)], dtype, "decode from token 0")
    # the first tokens of a sequence: position 0 alone sees only itself
    got = helpers.replay(s, helpers.trace_portions("f", ids[:5], (1, 1, 3)))
    helpers.check_against_plain(m, got, [("f", ids[:5])], dtype, "first tokens")


BENCH_SIZES = {   # the layer sizes of the models that the benchmark runs, two layers of each
    "124m": dict(n_embd=768, n_head=12),
    "355m": dict(n_embd=1024, n_head=16),       # the width at which the fused norm + product kernel ends
    "1.5b": dict(n_embd=1600, n_head=25),
}


@pytest.fixture(scope="module", params=sorted(BENCH_SIZES))
def bench_model(request, tmp_path_factory):
    size = request.param
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, vocab_size=50257, n_positions=1024,
               layer_norm_epsilon=1e-5, activation_function="gelu_new", bos_token_id=50256, eos_token_id=50256,
               **BENCH_SIZES[size])
    return helpers.make_model(tmp_path_factory.mktemp("bench_" + size.replace(".", "_")), cfg, seed=5)


@pytest.mark.parametrize("mode", ["whole", "bulk+single", "portions", "mixed"])
def test_layer_sizes_of_the_benchmark_models(bench_model, mode):
    """GPT-2 124M, 355M and 1.5B layer sizes (width, heads of 64, 4x inner width, the vocabulary of
    50,257 that is no multiple of anything, 1,024 positions), two layers, against the plain model, in
    32-bit and in bfloat16, each way of cutting: a request of 200 tokens (several key tiles, pages in
    any order) whole; most of it in one step and the last 32 tokens one by one; in portions of changing
    size; and cut into portions and single tokens beside a second request."""
    m = bench_model
    helpers.skip_in_simulation_if(True)
    reqs = [("long", m.prompt(200)), ("short", m.prompt(75, salt=1))]
    if mode == "whole":
        steps = helpers.trace_whole(*reqs[0])
    elif mode == "bulk+single":
        steps = helpers.trace_bulk_then_single(*reqs[0], 32)
    elif mode == "portions":
        steps = helpers.trace_portions(*reqs[0], sizes=(67, 2, 33, 5, 16, 3))
    else:
        steps = helpers.trace_mixed(reqs, seed=3, max_live=2, prefill_sizes=(130, 2, 37, 64), decode_tail=6)
    used = reqs if mode == "mixed" else reqs[:1]
    for dtype in DTYPES:
        s = session_for(m, dtype, max(helpers.max_live_tokens(steps), 256))
        got = helpers.replay(s, steps)
        helpers.check_against_plain(m, got, used, dtype, f"{m.cfg['n_embd']} wide, {mode}")
        s.cache.manager.check()


@pytest.mark.parametrize("page_size", [16, 32, 64])
def test_page_sizes(model_b, page_size):
    m = model_b
    ids = m.prompt(88)
    for dtype in DTYPES:
        s = session_for(m, dtype, 128, page_size)
        got = helpers.replay(s, helpers.trace_portions("p", ids, (15, 2, 33, 1)))
        helpers.check_against_plain(m, got, [("p", ids)], dtype, f"page {page_size}")


def test_want_subset_and_order(model_a):
    """Only the wanted rows come back, in the order of the entries and of `want`."""
    m = model_a
    a, b = m.prompt(12, 1), m.prompt(9, 2)
    s = session_for(m, "float32", 128)
    out = s.run_step({"step": 0, "entries": [{"id": "a", "tokens": a, "want": [11, 3]},
                                             {"id": "b", "tokens": b[:1], "want": []},
                                             ], "end": []})
    assert out.shape == (2, 512)
    ref = m.plain_logits(a)
    assert np.abs(out[0] - ref[11]).max() < 5e-6 and np.abs(out[1] - ref[3]).max() < 5e-6
    out = s.run_step({"step": 1, "entries": [{"id": "b", "tokens": b[1:], "want": [7]},
                                             {"id": "c", "tokens": a[:1], "want": [0]}], "end": ["a", "b", "c"]})
    assert np.abs(out[0] - m.plain_logits(b)[8]).max() < 5e-6
    assert np.abs(out[1] - ref[0]).max() < 5e-6
    assert s.run_step({"step": 2, "entries": [{"id": "z", "tokens": a, "want": []}], "end": ["z"]}) is None


def test_errors_leave_the_cache_as_it_was(model_a):
    from deliverance_amd.cache import OutOfPages
    from deliverance_amd.engine import StepError
    m = model_a
    s = session_for(m, "float32", 64)
    with pytest.raises(StepError, match="outside the vocabulary"):
        s.run_step({"step": 0, "entries": [{"id": "a", "tokens": [512], "want": []}], "end": []})
    with pytest.raises(StepError, match="the model has 128"):
        s.run_step({"step": 0, "entries": [{"id": "a", "tokens": [1] * 129, "want": []}], "end": []})
    with pytest.raises(OutOfPages):
        s.run_step({"step": 0, "entries": [{"id": "a", "tokens": [1] * 40, "want": []},
                                           {"id": "b", "tokens": [1] * 40, "want": []}], "end": []})
    s.cache.manager.check()
    assert s.cache.manager.live() == [] and s.cache.manager.pools[0].n_free == 4


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", DTYPES)
def test_bin_trace_run(model_b, dtype, tmp_path):
    """The program itself: steps on stdin, `done <step>` lines, <step>.f32 files."""
    m = model_b
    reqs = [("a", m.prompt(33)), ("b", m.prompt(9))]
    steps = helpers.trace_mixed(reqs, seed=1, decode_tail=4)
    out = tmp_path / "out"
    root = os.path.normpath(os.path.join(os.path.dirname(__file__), ".."))
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", m.folder, "--dtype", dtype,
                        "--out", str(out), "--max-tokens", str(helpers.max_live_tokens(steps))],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split("\n")[:len(steps)] == [f"done {s['step']}" for s in steps]
    got = {}
    V = m.cfg["vocab_size"]
    for s in steps:
        n = sum(len(e["want"]) for e in s["entries"])
        if n == 0:
            assert not (out / f"{s['step']}.f32").exists()
            continue
        arr = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n, V)
        r = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(arr[r]); r += 1
    got = {k: np.stack(v) for k, v in got.items()}
    helpers.check_against_plain(m, got, reqs, dtype, "bin/trace_run")
