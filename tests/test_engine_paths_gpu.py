"""The paths that generation really takes, compared at the level of logits: decode steps padded to a
bucket and replayed from a recorded HIP graph; steps launched ahead of the running one, their tokens
taken on the device; the plain kernels in bfloat16 (``kernels="reference"``); a request cancelled
while a step holds a reservation for it; the named intermediates of the debug hook."""
import numpy as np
import pytest

import helpers
import plain_gpt2 as P

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]


def decode_trace(reqs, prefill_tail):
    """Prompts whole (all but each request's last ``prefill_tail[i]`` tokens), one request a step;
    then every live request brings one token a step, so that the decode batch shrinks as requests
    end: 9, 5, 4, 3, ... sequences cross the sizes at which a recorded step's bucket changes."""
    steps, pos = [], {}
    for (rid, ids), tail in zip(reqs, prefill_tail):
        n = len(ids) - tail
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": ids[:n], "want": list(range(n))}], "end": []})
        pos[rid] = n
    live = [rid for rid, _ in reqs]
    by = dict(reqs)
    while live:
        entries, ends = [], []
        for rid in live:
            entries.append({"id": rid, "tokens": [by[rid][pos[rid]]], "want": [0]})
            pos[rid] += 1
            if pos[rid] == len(by[rid]):
                ends.append(rid)
        steps.append({"step": len(steps), "entries": entries, "end": ends})
        live = [r for r in live if r not in ends]
    return steps


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "B32"])
def test_decode_steps_padded_and_replayed_from_a_graph(models, name, dtype):
    """What ``generate`` runs for a decode step (the step padded with empty sequences to a power of
    two, block tables as wide as the longest context allows, tokens sampled on the device inside the
    recorded graph) gives the plain model's logits at every position; batches of 9, 5, 4, 3, 2, 1."""
    m = models[name]
    P_ = m.cfg["n_positions"]
    # lengths: one ends exactly at a page's end (32, 64), one at a page's start (17, 33), one uses the whole context
    lengths = [32, 17, 64, 33, 9, 40, 21, 50, min(P_, 90)]
    tails = [3, 5, 9, 14, 6, 20, 11, 25, 30]
    reqs = [(f"g{i}", m.prompt(n, salt=20 + i)) for i, n in enumerate(lengths)]
    steps = decode_trace(reqs, tails)
    sizes = {len(s["entries"]) for s in steps if all(len(e["tokens"]) == 1 for e in s["entries"])}
    assert {9, 5, 4, 3}.issubset(sizes), sizes
    s = helpers.trace_session(m.folder, dtype, 1024, poison_freed=True, use_graphs=True, sample=True)
    got, picked = {}, []
    for st in steps:
        out = s.run_step(st)
        r = 0
        for e in st["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(out[r]); r += 1
        if s.last_sampled is not None:
            assert s.last_sampled == [int(np.argmax(row)) for row in out], "the graph samples what its logits say"
            picked.append(len(s.last_sampled))
    assert len(s.runner._graphs) >= 4 and sum(picked) == sum(tails)       # buckets 1, 2, 4, 8, 16
    helpers.check_against_plain(m, {k: np.stack(v) for k, v in got.items()}, reqs, dtype, "graph decode")
    # a finished request's pages and a bucket's buffers are used again by the next request
    again = [("h0", m.prompt(40, salt=99)), ("h1", m.prompt(23, salt=98))]
    got = helpers.replay(s, decode_trace(again, [10, 10]))
    helpers.check_against_plain(m, got, again, dtype, "graph decode, second round")
    s.cache.manager.check()
    assert s.cache.manager.live() == []


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype,graphs", [("float32", True), ("bfloat16", True), ("bfloat16", False)])
def test_logits_of_steps_launched_ahead(models, dtype, graphs):
    """Generation itself (scheduler, steps launched ahead of the running one, tokens taken on the device,
    recorded graphs): the logits every step sampled from equal the plain model's at that position of the
    sequence that was generated."""
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    m = models["B"]
    prompts = [m.prompt(n, salt=40 + i) for i, n in enumerate((4, 30, 11, 2, 50, 23, 17))]
    params = [GeneratorParameters(max_tokens=k, ignore_eos=True) for k in (20, 5, 33, 40, 9, 17, 26)]
    eng = AutoModelForCausalLM.from_pretrained(m.folder, dtype=dtype, max_cached_tokens=1024, max_num_seqs=8,
                                               use_graphs=graphs, run_ahead=True, max_batch_tokens=48, max_chunk=16)
    seen = []     # (request index, position, logits row)

    def hook(batch, logits):
        rows = logits.detach().float().cpu().numpy()
        r = 0
        for sch in batch:
            if sch.samples:
                seen.append((sch.request.rid, sch.start + sch.n - 1, rows[r].copy()))
                r += 1
    eng.logits_hook = hook
    outs = eng.generate(prompts, params)
    assert eng.scheduler.counters["steps"] > 30
    by = {}
    for rid, pos, row in seen:
        by.setdefault(rid, {})[pos] = row
    rids = sorted(by)
    assert len(rids) == len(prompts)
    for rid, prompt, out in zip(rids, prompts, outs):
        ids = list(prompt) + out.generated_tokens
        positions = sorted(by[rid])
        assert positions == list(range(len(prompt) - 1, len(ids) - 1)), "one sampled row per generated token"
        got = np.stack([by[rid][p] for p in positions])
        helpers.check_against_plain(m, {rid: got}, [(rid, ids)], dtype, f"run-ahead graphs={graphs}", rows={rid: positions})


@pytest.mark.parametrize("name", ["A", "B32"])
def test_plain_kernels_in_bfloat16(models, name):
    """``kernels="reference"``: bfloat16 through the plain product and attention kernels, every way of
    cutting.  A mismatch that shows with the serving kernels and not here is theirs; one that shows in
    both is bfloat16's."""
    m = models[name]
    reqs = [(f"k{i}", m.prompt(n, salt=60 + i)) for i, n in enumerate((40, 17, 56, 9))]
    for what, steps in (("whole", helpers.trace_whole(*reqs[0])), ("bulk+single", helpers.trace_bulk_then_single(*reqs[0], 32)),
                        ("portions", helpers.trace_portions(*reqs[0])), ("mixed", helpers.trace_mixed(reqs, seed=2))):
        s = helpers.trace_session(m.folder, "bfloat16", 256, poison_freed=True, kernels="reference")
        got = helpers.replay(s, steps)
        helpers.check_against_plain(m, got, reqs if what == "mixed" else reqs[:1], "bfloat16", f"reference kernels, {what}")
    with pytest.raises(ValueError, match="kernels must be one of"):
        helpers.trace_session(m.folder, "bfloat16", 256, kernels="fast")


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", DTYPES)
def test_cancel_while_a_step_holds_a_reservation(models, dtype):
    """A request is cancelled between two steps, while a step launched ahead still runs for it and
    holds positions reserved for it: its pages come back at once, the others' tokens do not change,
    nothing is lost (the reference stops between tokens: GenerationEngine.java:221-225)."""
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    m = models["A"]
    prompts = [m.prompt(n, salt=70 + i) for i, n in enumerate((20, 9, 33, 14))]
    params = GeneratorParameters(max_tokens=30, ignore_eos=True)

    def engine():
        return AutoModelForCausalLM.from_pretrained(m.folder, dtype=dtype, max_cached_tokens=512, max_num_seqs=8,
                                                    run_ahead=True, poison_freed_pages=True)
    want = [o.generated_tokens for o in engine().generate(prompts, params)]
    eng = engine()
    rids = [eng.add_request(p, params) for p in prompts]
    done = {}
    for _ in range(12):
        for r in eng.step():
            done[r.rid] = r
    victim = rids[2]
    flight = eng._inflight
    assert flight is not None and any(s.request.rid == victim for s in flight.batch), "a step is running for the request"
    assert eng.cache.manager.pending(victim) >= 1, "and holds a reservation for it"
    free_before = eng.cache.manager.pools[0].n_free
    assert eng.cancel(victim) and not eng.cancel(victim)
    assert victim not in eng.cache.manager and eng.cache.manager.pools[0].n_free > free_before
    while eng.has_work():
        for r in eng.step():
            done[r.rid] = r
    for r in eng.drain():
        done[r.rid] = r
    assert done[victim].finish_reason == "cancelled" and 0 < len(done[victim].output) < 30
    assert done[victim].output == want[2][:len(done[victim].output)]
    for i in (0, 1, 3):
        if dtype == "float32":
            assert done[rids[i]].output == want[i]
        assert len(done[rids[i]].output) == 30 and done[rids[i]].finish_reason == "length"
    eng.cache.manager.check()
    assert eng.cache.manager.live() == [] and eng.cache.manager.pools[0].n_free == eng.cache.n_pages
    # a waiting request can be cancelled as well, and generate() reports a cancelled request
    eng2 = engine()
    box = {}

    def on_token(tok, i, ms):
        if i == 1 and box.get("n", 0) == 3:
            eng2.cancel(box["rids"][1])
        if i == 1:
            box["n"] = box.get("n", 0) + 1
    box["rids"] = list(range(len(prompts)))          # generate() numbers its requests from the engine's counter
    outs = eng2.generate(prompts, params, on_token=on_token)
    assert outs[1].finish_reason == "cancelled" and len(outs[1].generated_tokens) == 4
    assert [o.finish_reason for i, o in enumerate(outs) if i != 1] == ["length"] * 3
    assert eng2.cache.manager.pools[0].n_free == eng2.cache.n_pages


@pytest.mark.parametrize("dtype", DTYPES)
def test_named_intermediates_of_a_step(models, dtype):
    """The debug hook hands out (layer, stage, tensor) as the reference's does
    (AbstractModel.java:122-128,1100-1107; TransformerBlock.java:177,189; CausalSelfAttention.java:299-301,384,406):
    each against the plain model's value at that place."""
    m = models["B"]
    cfg, W = m.plain_cfg, m.W
    ids = m.prompt(37, salt=5)
    s = helpers.trace_session(m.folder, dtype, 128)
    seen = {}
    s.runner.debug_hook = lambda layer, stage, t: seen.setdefault((layer, stage), t.float().cpu().numpy())
    helpers.replay(s, [{"step": 0, "entries": [{"id": "d", "tokens": ids[:30], "want": []}], "end": []},
                       {"step": 1, "entries": [{"id": "d", "tokens": ids[30:], "want": [6]}], "end": ["d"]}])
    # the hook saw the first step (30 rows); the plain model's rows of the same positions
    x = P.embed(ids[:30], list(range(30)), W["wte.weight"], W["wpe.weight"])
    tol = 2e-5 if dtype == "float32" else 6e-2
    assert np.abs(seen[(-1, "input")] - x).max() < (1e-6 if dtype == "float32" else 1e-6)
    H, D = cfg["n_head"], cfg["n_embd"] // cfg["n_head"]
    for layer in range(cfg["n_layer"]):
        a = P.layer_norm(x, W[f"h.{layer}.ln_1.weight"], W[f"h.{layer}.ln_1.bias"], cfg["layer_norm_epsilon"])
        qkv = P.conv1d(a, W[f"h.{layer}.attn.c_attn.weight"], W[f"h.{layer}.attn.c_attn.bias"])
        E = cfg["n_embd"]
        for k, stage in enumerate(("query_projection", "key_projection", "value_projection")):
            assert np.abs(seen[(layer, stage)] - qkv[:, k * E:(k + 1) * E]).max() < tol, (layer, stage)
        scale = 1.0 / np.sqrt(D) / ((layer + 1) if cfg.get("scale_attn_by_inverse_layer_idx") else 1)
        att = P.causal_attention(qkv[:, :E], qkv[:, E:2 * E], qkv[:, 2 * E:], H, scale)
        assert np.abs(seen[(layer, "attention_value")] - att).max() < tol, layer
        # the output projection before its bias (CausalSelfAttention.java:406)
        assert np.abs(seen[(layer, "attention_output")] - att @ W[f"h.{layer}.attn.c_proj.weight"]).max() < tol, layer
        x1 = x + P.conv1d(att, W[f"h.{layer}.attn.c_proj.weight"], W[f"h.{layer}.attn.c_proj.bias"])
        assert np.abs(seen[(layer, "post_attention_residual")] - x1).max() < tol, layer
        x = P.block(x, W, layer, cfg)
        assert np.abs(seen[(layer, "post_ff_residual")] - x).max() < tol, layer
        assert np.abs(seen[(layer, "layer_output")] - x).max() < tol, layer
    assert len(seen) == 1 + 8 * cfg["n_layer"]


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """2,304 positions: decode attention shares a sequence's keys out over two workgroups a head."""
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=128, n_head=2, vocab_size=300,
               n_positions=2304, layer_norm_epsilon=1e-5, activation_function="gelu_new", bos_token_id=0, eos_token_id=1)
    return helpers.make_model(tmp_path_factory.mktemp("long"), cfg, seed=9)


@pytest.mark.parametrize("graphs", [False, True])
def test_decoding_over_a_long_context(long_model, graphs):
    """A context of 2,200 tokens and one of 1,100 beside it, the last 24 tokens one by one: the decode
    kernel splits the keys over workgroups (the block table spans more than 2,048 keys) and merges."""
    from deliverance_amd.kernels import ops
    m = long_model
    helpers.skip_in_simulation_if(True)
    reqs = [("far", m.prompt(2200, salt=1)), ("near", m.prompt(1100, salt=2))]
    steps = decode_trace(reqs, [24, 24])
    assert ops.decode_splits(2, 2, -(-2200 // 16), 16) == 2
    s = helpers.trace_session(m.folder, "bfloat16", 4096, poison_freed=True, use_graphs=graphs, sample=graphs)
    got = helpers.replay(s, steps)
    helpers.check_against_plain(m, got, reqs, "bfloat16", f"long context, graphs={graphs}")
    if graphs:
        assert s.runner._graphs
