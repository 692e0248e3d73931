"""The models that the benchmark runs, at their full depth: GPT-2 124M (12 layers), 355M (24) and 1.5B
(48), random weights written by the random-weights mode and read back by the engine's own loader (a
checkpoint of 3 GB for the largest), against the plain model, in 32-bit and in bfloat16.

bfloat16 error grows with depth, and a 32-bit sum over a width of 1,600 in 48 layers is not the sum over
64 in 2: the bounds that the tiny configurations are held to are held here too.  One request of 200
tokens is replayed whole; then cut into portions and single tokens beside a second request, with so few
pages that they are used again; then generation itself runs at the largest size, its decode steps
replayed from recorded graphs and launched ahead, with batches that cross the buckets of 64 down to 1
(the reference's counterpart compares cached decoding with a cold replay:
core/src/test/java/io/teknek/deliverance/model/hf/HfGenerationTesterMixinPort.java:16-36)."""
import numpy as np
import pytest

import helpers

pytestmark = [pytest.mark.gpu, pytest.mark.needs_device]

FULL = {
    "124m": dict(n_layer=12, n_embd=768, n_head=12),
    "355m": dict(n_layer=24, n_embd=1024, n_head=16),
    "1.5b": dict(n_layer=48, n_embd=1600, n_head=25),
}


@pytest.fixture(scope="module", params=["124m", "355m", "1.5b"])
def full_model(request, tmp_path_factory):
    size = request.param
    cfg = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", vocab_size=50257, n_positions=1024,
               layer_norm_epsilon=1e-5, activation_function="gelu_new", bos_token_id=50256, eos_token_id=50256, **FULL[size])
    print(f"[full depth] writing and reading GPT-2 {size} ({cfg['n_layer']} layers)", flush=True)
    m = helpers.make_model(tmp_path_factory.mktemp("full_" + size.replace(".", "_")), cfg, seed=11)
    m.size = size
    yield m
    m.W = None          # (the plain model's 64-bit copy of the weights: 12 GB at the largest size)


@pytest.mark.parametrize("mode", ["whole", "mixed"])
def test_full_depth_against_the_plain_model(full_model, mode):
    m = full_model
    reqs = [("long", m.prompt(200)), ("short", m.prompt(75, salt=1))]
    if mode == "whole":
        steps, used = helpers.trace_whole(*reqs[0]), reqs[:1]
    else:
        steps, used = helpers.trace_mixed(reqs, seed=3, max_live=2, prefill_sizes=(130, 2, 37, 64), decode_tail=6), reqs
        assert any(len({len(e["tokens"]) == 1 for e in s["entries"]}) == 2 for s in steps)   # portions beside single tokens
    for dtype in ("float32", "bfloat16"):
        print(f"[full depth] {m.size} {mode} {dtype}", flush=True)
        s = helpers.trace_session(m.folder, dtype, helpers.max_live_tokens(steps), poison_freed=True)
        got = helpers.replay(s, steps)
        helpers.check_against_plain(m, got, used, dtype, f"GPT-2 {m.size} at full depth, {mode}")
        if mode == "mixed":       # a third request into the pages that the first two gave back
            again = [("again", m.prompt(90, salt=2))]
            got = helpers.replay(s, helpers.trace_portions(*again[0], sizes=(50, 2, 30, 1)))
            helpers.check_against_plain(m, got, again, dtype, f"GPT-2 {m.size} at full depth, pages used again")
        s.cache.manager.check()
        assert s.cache.manager.live() == []
        del s


def test_generation_at_full_depth_graphs_and_steps_launched_ahead(full_model):
    """``generate()`` at GPT-2 1.5B's size: 40 requests at once (a decode batch in the bucket of 64), ending
    at different lengths so that the batch falls through the buckets of 32, 16, 8, ... 1; every step's
    logits, as the sampler saw them, against the plain model at that position of the generated sequence."""
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    m = full_model
    if m.size != "1.5b":
        pytest.skip("run once, at the largest size")
    n_req = 40
    prompts = [m.prompt(3 + (5 * i) % 11, salt=100 + i) for i in range(n_req)]
    params = [GeneratorParameters(max_tokens=2 + (7 * i) % 13 if i % 5 else 14 + i // 5, ignore_eos=True) for i in range(n_req)]
    eng = AutoModelForCausalLM.from_pretrained(m.folder, dtype="bfloat16", max_cached_tokens=64 * 64, max_num_seqs=64,
                                               use_graphs=True, run_ahead=True, max_batch_tokens=512, max_chunk=256)
    seen, batches = [], set()

    def hook(batch, logits):
        rows = logits.detach().float().cpu().numpy()
        if all(sch.n == 1 for sch in batch):
            batches.add(len(batch))
        r = 0
        for sch in batch:
            if sch.samples:
                seen.append((sch.request.rid, sch.start + sch.n - 1, rows[r].copy()))
                r += 1
    eng.logits_hook = hook
    print("[full depth] generating", flush=True)
    outs = eng.generate(prompts, params)
    assert eng.runner._graphs and {64, 8}.issubset(eng.runner._graphs), sorted(eng.runner._graphs)
    assert any(b > 32 for b in batches) and any(b <= 8 for b in batches), sorted(batches)
    by = {}
    for rid, pos, row in seen:
        by.setdefault(rid, {})[pos] = row
    rids = sorted(by)
    assert len(rids) == n_req
    print("[full depth] comparing with the plain model", flush=True)
    for rid, prompt, out in zip(rids, prompts, outs):
        ids = list(prompt) + out.generated_tokens
        positions = sorted(by[rid])
        assert positions == list(range(len(prompt) - 1, len(ids) - 1)), "one sampled row per generated token"
        got = np.stack([by[rid][p] for p in positions])
        helpers.check_against_plain(m, {rid: got}, [(rid, ids)], "bfloat16", "generation at full depth",
                                    rows={rid: positions})
