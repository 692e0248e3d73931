"""Generation through the entry point: greedy against the plain implementation, seeded
temperature sampling, the stop rules, what happens when pages run out, and the replayed-graph
decode against the step-by-step one."""
import numpy as np
import pytest

import helpers
import plain_gpt2 as P

pytestmark = pytest.mark.gpu


def load(model, dtype="float32", **kw):
    from deliverance_amd import AutoModelForCausalLM
    kw.setdefault("max_cached_tokens", 1024)
    kw.setdefault("max_num_seqs", 8)
    return AutoModelForCausalLM.from_pretrained(model.folder, dtype=dtype, **kw)


@pytest.mark.parametrize("name,lengths,n_new", [("A", (5, 17, 40), 16), ("B", (1, 9, 33, 64), 24)])
def test_greedy_equals_the_plain_model(models, name, lengths, n_new):
    from deliverance_amd import GeneratorParameters
    m = models[name]
    prompts = [m.prompt(n) for n in lengths]
    eng = load(m, "float32")
    outs = eng.generate(prompts, GeneratorParameters(max_tokens=n_new, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        assert out.generated_tokens == P.greedy_generate(m.plain_cfg, m.W, prompt, n_new)
        assert out.finish_reason == "length" and out.prompt_tokens == len(prompt)
        assert out.total_time_ms >= out.time_to_first_token_ms > 0
    eng.cache.manager.check()
    assert eng.cache.manager.live() == []
    # one prompt alone gives what it gave in the batch
    alone = eng.generate(prompts[1], GeneratorParameters(max_tokens=n_new, ignore_eos=True))
    assert alone.generated_tokens == outs[1].generated_tokens


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_in_bfloat16_stays_within_rounding_of_the_plain_maximum(models, name):
    from deliverance_amd import GeneratorParameters
    m = models[name]
    prompts = [m.prompt(n) for n in (9, 33)]
    for graphs in (True, False):
        eng = load(m, "bfloat16", use_graphs=graphs)
        outs = eng.generate(prompts, GeneratorParameters(max_tokens=12, ignore_eos=True))
        for prompt, out in zip(prompts, outs):
            ids = list(prompt)
            for t in out.generated_tokens:
                lg = m.plain_logits(ids)[-1]
                assert lg[t] >= lg.max() - helpers.bf16_token_slack(lg)
                ids.append(t)


def test_replayed_graph_decodes_what_the_step_by_step_path_decodes(model_b):
    from deliverance_amd import GeneratorParameters
    m = model_b
    prompts = [m.prompt(n, salt=3) for n in (4, 30, 11, 2, 50)]
    params = [GeneratorParameters(max_tokens=k, ignore_eos=True) for k in (20, 5, 33, 40, 9)]   # batches shrink as requests end
    outs = {}
    for graphs in (True, False):
        eng = load(m, "bfloat16", use_graphs=graphs)
        outs[graphs] = [o.generated_tokens for o in eng.generate(prompts, params)]
        assert bool(eng.runner._graphs) == graphs
    assert outs[True] == outs[False]


@pytest.mark.parametrize("dtype,graphs", [("bfloat16", True), ("float32", False)])
def test_steps_launched_ahead_decode_what_steps_read_one_by_one_decode(model_b, dtype, graphs):
    """With run_ahead the next decode step is launched before the running one's tokens are read
    (they are taken on the device); requests that end by length leave the batch in time, a request
    that samples an end token has one step too many, whose result is dropped."""
    from deliverance_amd import GeneratorParameters
    m = model_b
    prompts = [m.prompt(n, salt=7) for n in (4, 30, 11, 2, 50, 23)]
    eng0 = load(m, dtype, use_graphs=graphs, run_ahead=False)
    free = eng0.generate(prompts[3], GeneratorParameters(max_tokens=40, ignore_eos=True)).generated_tokens
    eos = {free[10]}
    params = [GeneratorParameters(max_tokens=20, ignore_eos=True), GeneratorParameters(max_tokens=5, ignore_eos=True),
              GeneratorParameters(temperature=0.9, seed=77, top_k=40, max_tokens=33, ignore_eos=True),
              GeneratorParameters(max_tokens=40), GeneratorParameters(ntokens=59, ignore_eos=True),
              GeneratorParameters(temperature=0.7, seed=3, top_p=0.9, max_tokens=17, ignore_eos=True)]
    outs = {}
    for ahead in (False, True):
        eng = load(m, dtype, use_graphs=graphs, run_ahead=ahead)
        eng.scheduler.eos = eos
        seen = []
        res = eng.generate(prompts, params, on_token=lambda tok, i, ms: seen.append((i, tok)))
        outs[ahead] = [(o.generated_tokens, o.finish_reason) for o in res]
        for i, o in enumerate(res):
            assert [t for j, t in seen if j == i] == o.generated_tokens
        assert eng._inflight is None and not eng.has_work()
        eng.cache.manager.check()
        assert eng.cache.manager.live() == []
        if ahead:
            assert eng.scheduler.counters["steps"] > 0
    assert outs[True] == outs[False]
    assert outs[True][3] == (free[:free.index(free[10]) + 1], "stop")
    assert [len(t) for t, _ in outs[True]] [:3] == [20, 5, 33] and len(outs[True][4][0]) == 59 + 1 - 50


def test_temperature_sampling_is_seeded_and_matches_the_plain_sampler(model_b):
    """Config B's workload: temperature 0.8, 24 tokens, a fixed seed."""
    from deliverance_amd import GeneratorParameters
    m = model_b
    prompt = m.prompt(33)
    eng = load(m, "float32")
    for kw in (dict(), dict(top_k=50), dict(top_p=0.9), dict(top_k=20, top_p=0.7, uniform_top_p=1.0)):
        params = GeneratorParameters(temperature=0.8, seed=1234, max_tokens=24, ignore_eos=True, **kw)
        out = eng.generate(prompt, params)
        rng = P.JavaRandom(1234)
        ids = list(prompt)
        for _ in range(24):
            rng.next_float()                                  # the draw made with the sampler
            u = rng.next_float()
            ids.append(P.sample_top_k_top_p(m.plain_logits(ids)[-1], 0.8, kw.get("top_k"), kw.get("top_p"),
                                            kw.get("uniform_top_p"), u))
        assert out.generated_tokens == ids[len(prompt):], kw
        # the same request among others gives the same tokens: its random stream is its own
        others = [m.prompt(9), prompt, m.prompt(17)]
        plist = [GeneratorParameters(temperature=1.1, seed=5, max_tokens=30, ignore_eos=True), params,
                 GeneratorParameters(max_tokens=10, ignore_eos=True)]
        assert eng.generate(others, plist)[1].generated_tokens == out.generated_tokens
    a = eng.generate(prompt, GeneratorParameters(temperature=0.8, seed=1, max_tokens=24, ignore_eos=True))
    b = eng.generate(prompt, GeneratorParameters(temperature=0.8, seed=2, max_tokens=24, ignore_eos=True))
    assert a.generated_tokens != b.generated_tokens


def test_stop_rules(model_a):
    from deliverance_amd import GeneratorParameters
    from deliverance_amd.engine import SchedulerError
    m = model_a
    eng = load(m, "float32")
    prompt = m.prompt(17)
    free = P.greedy_generate(m.plain_cfg, m.W, prompt, 30)
    # max_tokens: exactly that many (the reference: MaxTokenTest.java:113-121)
    assert len(eng.generate(prompt, GeneratorParameters(max_tokens=8, ignore_eos=True)).generated_tokens) == 8
    # ntokens bounds positions: 17 + generated = ntokens + 1
    out = eng.generate(prompt, GeneratorParameters(ntokens=25, ignore_eos=True))
    assert out.finish_reason == "length" and len(out.generated_tokens) == 25 + 1 - 17
    # without limits the context ends the request
    out = eng.generate(prompt, GeneratorParameters(ignore_eos=True))
    assert len(prompt) + len(out.generated_tokens) == m.cfg["n_positions"] + 1
    # an end token stops and is counted; it is the model's eos id (511 in config A): make it appear by hand
    import dataclasses
    eng.scheduler.eos = {free[4]}
    out = eng.generate(prompt, GeneratorParameters(max_tokens=30))
    first = free.index(free[4])
    assert out.finish_reason == "stop" and out.generated_tokens == free[:first + 1]
    with pytest.raises(SchedulerError, match="Prompt exceeds ntokens"):
        eng.generate(m.prompt(128), GeneratorParameters())
    with pytest.raises(ValueError, match="outside the vocabulary"):
        eng.generate([1, 2, 512], GeneratorParameters())
    eng.cache.manager.check()
    assert eng.cache.manager.live() == []


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_when_pages_run_out_requests_are_computed_again_with_the_same_result(model_a, dtype):
    from deliverance_amd import GeneratorParameters
    m = model_a
    prompts = [m.prompt(n, salt=9) for n in (40, 23, 31, 12)]
    params = GeneratorParameters(max_tokens=40, ignore_eos=True)
    roomy = load(m, dtype, max_cached_tokens=1024)
    want = [o.generated_tokens for o in roomy.generate(prompts, params)]
    tight = load(m, dtype, max_cached_tokens=192, max_batch_tokens=48, max_chunk=16,     # 12 pages for ~270 tokens
                 poison_freed_pages=True)      # and what a request that is set back gives up is NaN again
    outs = tight.generate(prompts, params)
    assert sum(o.preemptions for o in outs) >= 1 and tight.stats()["preemptions"] >= 1
    if dtype == "float32":
        assert [o.generated_tokens for o in outs] == want
    else:
        # bfloat16 rounds differently when a prompt is cut differently: every token must still be a
        # maximum of the plain logits within rounding
        for prompt, out in zip(prompts, outs):
            ids = list(prompt)
            for t in out.generated_tokens:
                lg = m.plain_logits(ids)[-1]
                assert lg[t] >= lg.max() - helpers.bf16_token_slack(lg)
                ids.append(t)
    tight.cache.manager.check()
    assert tight.cache.manager.pools[0].n_free == tight.cache.n_pages
    # a request that cannot fit even alone fails with a clear reason
    tiny = load(m, dtype, max_cached_tokens=32)
    out = tiny.generate(m.prompt(20), GeneratorParameters(max_tokens=60, ignore_eos=True))
    assert out.finish_reason == "error" and "more cache than the whole pool" in out.error
    assert tiny.cache.manager.pools[0].n_free == tiny.cache.n_pages


def test_callbacks_and_logprobs(model_a):
    from deliverance_amd import GeneratorParameters
    m = model_a
    eng = load(m, "float32")
    seen = []
    prompts = [m.prompt(5), m.prompt(9)]
    outs = eng.generate(prompts, GeneratorParameters(max_tokens=4, ignore_eos=True, log_probs=True, top_log_probs=3),
                        on_token=lambda tok, idx, ms: seen.append((idx, tok)))
    for i, out in enumerate(outs):
        assert [t for j, t in seen if j == i] == out.generated_tokens
        assert len(out.top_logprobs) == 4
        ids = list(prompts[i])
        for step, tok in enumerate(out.generated_tokens):
            lg = m.plain_logits(ids)[-1]
            lp = lg - np.log(np.exp(lg - lg.max()).sum()) - lg.max()
            top = np.argsort(-lp, kind="stable")[:3]
            got = out.top_logprobs[step]
            assert [g[0] for g in got] == [int(t) for t in top]
            assert np.abs(np.array([g[1] for g in got]) - lp[top]).max() < 1e-4
            ids.append(tok)


def test_command_line_generates_what_the_plain_model_generates(model_a, tmp_path):
    import json, os, subprocess, sys
    m = model_a
    prompts = [m.prompt(5), m.prompt(17)]
    root = os.path.normpath(os.path.join(os.path.dirname(__file__), ".."))
    suite = tmp_path / "suite.jsonl"
    suite.write_text(json.dumps({"prompt_ids": prompts[1]}) + "\n")
    out_csv, out_jsonl = tmp_path / "o.csv", tmp_path / "o.jsonl"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "deliverance"), "generate", "--model", m.folder,
                        "--working-dtype", "F32", "--prompt-ids", ",".join(map(str, prompts[0])), "--suite-file", str(suite),
                        "--max-tokens", "8", "--ignore-eos", "--temperature", "0.0", "--seed", "42", "--max-cached-tokens", "512",
                        "--profile-stages", "--output", str(out_csv), "--jsonl-output", str(out_jsonl)],
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.strip().split("\n") if l]
    for prompt, line in zip(prompts, lines):
        assert [int(t) for t in line.split(",")] == P.greedy_generate(m.plain_cfg, m.W, prompt, 8)
    assert p.stderr.count("generation_complete prompt_tokens=") == 2 and "finish_reason=length" in p.stderr
    assert "generation.decode" in p.stderr and "profile summary" in p.stderr
    assert out_csv.read_text().split("\n")[0] == "prompt_tokens,generated_tokens,total_ms,generation_ms,tokens_per_second"
    rec = [json.loads(l) for l in out_jsonl.read_text().strip().split("\n")]
    assert rec[1]["prompt_ids"] == prompts[1] and rec[1]["generated_tokens"] == 8
