#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens a second at a fixed batch, prefill of 2,048
tokens, and the decode step's fraction of the HBM roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model 124m|355m|1.5b] [--batch B]

A "step" is one decode step of the engine (scheduler decision, model step over the paged cache,
sampling on the device, tokens back on the host).  Weights are random (N(0, 0.02)), prompts are
seeded uniform-random token ids of 512 tokens, decoding is greedy and ignores end tokens.

The default run measures GPT-2 124M layer sizes (the headline `value`: batch 8; `points`: batch 1
and 64; `prefill`: one step of 2 x 1,024 tokens) and then, into the same line, GPT-2 1.5B layer
sizes (decode at batch 1, 8, 64 and the same prefill) and the mixed workload at GPT-2 355M layer
sizes (64 requests at once, prompt portions of 512 tokens beside the others' decoding), each with
its fraction of the roofline; `--no-extra` leaves those two out.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# GPT-2 layer sizes (random weights; n_positions 1024, vocabulary 50257, tied head)
MODELS = {
    "124m": dict(n_layer=12, n_embd=768, n_head=12),
    "355m": dict(n_layer=24, n_embd=1024, n_head=16),
    "1.5b": dict(n_layer=48, n_embd=1600, n_head=25),
}
# MI355X published peaks
HBM_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
SETTLE_STEPS = 3        # decode steps before the warm-up: the first records the step's HIP graph


def model_config(name, n_layer=None, n_positions=1024):
    c = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", vocab_size=50257, n_positions=n_positions,
             layer_norm_epsilon=1e-5, activation_function="gelu_new", bos_token_id=50256, eos_token_id=50256)
    c.update(MODELS[name])
    if n_layer is not None:
        c["n_layer"] = n_layer
    return c


def weight_bytes(c, el):
    E, I, V, L = c["n_embd"], 4 * c["n_embd"], c["vocab_size"], c["n_layer"]
    per_layer = (3 * E * E + E * E + 2 * E * I) * el + (3 * E + E + I + E + 4 * E) * el
    return L * per_layer + V * E * el + 2 * E * el          # blocks + head table (read once) + ln_f


def step_flops(c, seq_lens_new, past=0):
    """Matrix-product and attention flops of a step that brings ``seq_lens_new`` tokens per sequence."""
    E, I, V, L = c["n_embd"], 4 * c["n_embd"], c["vocab_size"], c["n_layer"]
    n = sum(seq_lens_new)
    gemm = 2 * n * (3 * E * E + E * E + 2 * E * I) * L + 2 * len(seq_lens_new) * E * V
    attn = 0
    for t in seq_lens_new:
        keys = sum(past + i + 1 for i in range(t))
        attn += 4 * keys * E * L
    return gemm + attn


def decode_roofline(cfg, el, batch, ctx_mean, seconds_per_step):
    """Bytes a decode step must read (every weight once, the live requests' cache) over its time."""
    kv_bytes_per_token = 2 * cfg["n_embd"] * el * cfg["n_layer"]
    step_bytes = weight_bytes(cfg, el) + batch * ctx_mean * kv_bytes_per_token
    return step_bytes / seconds_per_step / 1e9


def engine_from_folder(folder, dtype, seats, cfg, **kw):
    from deliverance_amd import AutoModelForCausalLM
    kw.setdefault("max_batch_tokens", max(2048, seats))
    kw.setdefault("max_chunk", 1024)
    kw.setdefault("page_size", 16)
    return AutoModelForCausalLM.from_pretrained(folder, dtype=dtype, max_num_seqs=max(seats, 2),
                                                max_cached_tokens=max(seats, 2) * cfg["n_positions"], **kw)


def engine_from_gpu_weights(cfg, dtype, seats, seed=0, **kw):
    """The same engine with its random weights drawn on the GPU (the tensors that the architecture
    declares, with the standard deviations it declares for them), for the models whose checkpoint would
    take longer to write to disk and read back than to measure."""
    import torch
    import deliverance_amd.models  # noqa: F401
    from deliverance_amd import EngineConfig
    from deliverance_amd.engine.engine import CausalLanguageModel
    from deliverance_amd.models.causal_lm import CausalLM
    from deliverance_amd.registry import ModelSupport
    arch = ModelSupport.detect(cfg)
    mc = arch.read_config(cfg)
    g = torch.Generator(device="cuda:0")
    g.manual_seed(seed)
    tensors = {}
    for d in arch.declare_tensors(mc):
        if d.optional:
            continue
        t = torch.randn(d.shape, generator=g, device="cuda:0", dtype=torch.float32) * d.std
        if d.init == "ones_plus_normal":
            t += 1.0
        tensors[d.name] = t.to(torch.bfloat16)
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    model = CausalLM(mc, arch.bind_tensors(mc, tensors), tdt, "cuda:0")
    del tensors
    kw.setdefault("max_batch_tokens", max(2048, seats))
    kw.setdefault("max_chunk", 1024)
    kw.setdefault("page_size", 16)
    pool = kw.pop("max_cached_tokens", max(seats, 2) * cfg["n_positions"])
    ec = EngineConfig(dtype=dtype, max_num_seqs=max(seats, 2), max_cached_tokens=pool, **kw)
    return CausalLanguageModel(model, ec)


def decode_run(model, cfg, rng, batch, prompt_len, steps, warmup):
    """Prefill ``batch`` prompts and settle (untimed), ``warmup`` decode steps, then time ``steps`` decode
    steps.  The requests outlive the timed steps, so that none of them ends (and no smaller batch has its
    graph recorded) inside the timed region.  Returns (seconds, mean context length in the timed steps)."""
    import torch
    from deliverance_amd import GeneratorParameters
    # (requests admitted first decode while the others' prompts are still processed: one token a prefill step)
    stagger = -(-batch * prompt_len // model.engine_config.max_batch_tokens)
    total = stagger + SETTLE_STEPS + warmup + steps + 8
    assert prompt_len + total + 1 <= cfg["n_positions"], "prompt and decoded tokens exceed n_positions"
    params = GeneratorParameters(max_tokens=total, ignore_eos=True)
    rids = [model.add_request([int(t) for t in rng.integers(0, cfg["vocab_size"], size=prompt_len)], params)
            for _ in range(batch)]
    while any(r.n_computed < len(r.prompt) for r in model.scheduler.running) or model.scheduler.waiting:
        model.step()
    for _ in range(SETTLE_STEPS + warmup):
        model.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        model.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert len(model.scheduler.running) == batch, "a request ended inside the timed steps"
    ctx_mean = prompt_len + 1 + stagger / 2.0 + SETTLE_STEPS + warmup + steps / 2.0
    for rid in rids:
        model.cancel(rid)
    while model.has_work():
        model.step()
    model.drain()
    model.scheduler.finished.clear()
    return dt, ctx_mean


def prefill_run(model, cfg, rng, dkey, n_prompts=2, length=1024):
    """``n_prompts`` x ``length``-token prompts (2 x 1,024 unless asked otherwise) in ONE step of the engine's step
    function, logits at the last row of each."""
    import torch
    from deliverance_amd.engine.step import StepEntry
    times = []
    for it in range(5):                       # the first rounds warm up; the best of the rest counts
        entries = [StepEntry(f"prefill{i}", [int(t) for t in rng.integers(0, cfg["vocab_size"], size=length)], [length - 1])
                   for i in range(n_prompts)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.runner.run(entries)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        for e in entries:
            model.cache.manager.close(e.rid)
    t = min(times[2:])
    fl = step_flops(cfg, [length] * n_prompts)
    n = n_prompts * length
    return {"value": round(n / t, 1), "tokens": n, "ms": round(t * 1e3, 3), "frac": round(fl / t / PEAK_FLOPS[dkey], 4)}


def mixed_run(model, cfg, rng, n_req=64, new=128):
    """Continuous batching under load: every request arrives at once; the scheduler admits them as
    seats and pages allow, cuts prompts into portions of at most 512 tokens and runs them in the
    same steps as the other requests' decoding.  Run twice (the first run records the decode
    graphs): the two runs must generate the same tokens.  Returns a dict of what was measured."""
    import torch
    from deliverance_amd import GeneratorParameters
    longest = cfg["n_positions"] - new - 1
    lengths = [int(x) for x in rng.integers(16, longest + 1, size=n_req)]
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lengths]
    params = GeneratorParameters(max_tokens=new, ignore_eos=True)
    best, tokens = None, []
    for _ in range(2):
        before = model.stats()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = model.generate(prompts, params)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tokens.append([o.generated_tokens for o in outs])
        if best is None or dt < best:
            best = dt
            after = model.stats()
            steps = after["steps"] - before["steps"]
            batch_tokens = after["batch_tokens"] - before["batch_tokens"]
    assert all(len(t) == new for t in tokens[0])
    same = sum(a == b for a, b in zip(*tokens))
    return dict(value=round(n_req * new / best, 1), seconds=round(best, 4), prompt_tokens=sum(lengths),
                generated_tokens=n_req * new, all_tokens_per_second=round((sum(lengths) + n_req * new) / best, 1),
                steps=steps, mean_batch_tokens=round(batch_tokens / max(steps, 1), 1), longest_prompt=longest,
                requests_equal_in_both_runs=same, requests=n_req, preemptions=model.stats().get("preemptions", 0))


def kernel_table(model, cfg, rng, batch, prompt_len, n_prompts=2, length=1024):
    """--profile-stages: every kernel of a prefill step and of a few decode steps timed on the device,
    against the bytes it must move and the flops it must do (stderr)."""
    from deliverance_amd.profiler import KernelProfiler
    KernelProfiler.enable()
    prefill_run(model, cfg, rng, "bf16", n_prompts, length)
    print(KernelProfiler.summary(f"prefill, {n_prompts} x {length:,} tokens, 5 steps (% of 8 TB/s or of the matrix peak, whichever binds)"),
          file=sys.stderr)
    KernelProfiler.reset()
    decode_run(model, cfg, rng, batch, prompt_len, 16, 0)
    print(KernelProfiler.summary(f"prefill of {batch} x {prompt_len} tokens, then {SETTLE_STEPS + 16} decode steps at batch {batch}"),
          file=sys.stderr)
    KernelProfiler.disable()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="124m", choices=sorted(MODELS))
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--n-positions", type=int, default=1024, help="context length of the random model (GPT-2: 1,024)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--kernels", default="tuned", choices=["tuned", "reference"])
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the GPT-2 1.5B points and the 355M mixed workload")
    ap.add_argument("--profile-stages", action="store_true", help="also print a per-kernel table with roofline fractions (stderr)")
    ap.add_argument("--page-size", type=int, default=16, choices=[16, 32, 64], help="tokens a cache page")
    ap.add_argument("--prefill-shape", default="2x1024", help="prompts x tokens of the prefill step (the contract's: 2x1024)")
    ap.add_argument("--step-tokens", type=int, default=512 + 64,
                    help="mixed workload: the most tokens a step holds, decoded tokens and a prompt portion together (default: a portion of 512 beside 64 decoded tokens)")
    ap.add_argument("--pool-tokens", type=int, default=None,
                    help="mixed workload: tokens of cache the pool holds (default: every request at full length; fewer force "
                         "requests out of the cache and back, which the line reports as preemptions)")
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed"],
                    help="mixed: only the mixed workload, on --model (64 requests with prompts of 16 to 895 tokens arrive at "
                         "once, prompt portions of 512 tokens run beside the decoding of the others, 128 new tokens each)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import numpy as np
    from deliverance_amd.random_model import random_model

    cfg = model_config(args.model, args.layers, args.n_positions)
    full_layers = MODELS[args.model]["n_layer"]
    el = 2 if args.dtype == "bfloat16" else 4
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    rng = np.random.default_rng(0)
    pf_n, pf_len = (int(x) for x in args.prefill_shape.lower().split("x"))
    if not args.no_prefill and args.workload == "decode" and pf_len > cfg["n_positions"]:
        print(f"a prompt of {pf_len} tokens exceeds n_positions {cfg['n_positions']}")
        return 2
    if args.prompt_len + SETTLE_STEPS + args.warmup + args.steps + 9 > cfg["n_positions"]:
        print(f"prompt {args.prompt_len} + {SETTLE_STEPS + args.warmup + args.steps + 9} decoded tokens exceed n_positions {cfg['n_positions']}")
        return 2

    if args.workload == "mixed":
        model = engine_from_gpu_weights(cfg, args.dtype, 64, kernels=args.kernels, max_batch_tokens=args.step_tokens, max_chunk=512, page_size=args.page_size,
                                        **({"max_cached_tokens": args.pool_tokens} if args.pool_tokens else {}))
        m = mixed_run(model, cfg, rng)
        print(json.dumps({
            "metric": "generated tok/s, %d requests at once (GPT-2 %s layer sizes, prompts 16..%d, 128 new tokens each, "
                      "prompt portions of 512 beside decoding)" % (m["requests"], args.model, m["longest_prompt"]),
            "value": m["value"], "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True, "dtype": dkey,
            "data": "synthetic (random weights drawn on the GPU, uniform-random token ids)", **{k: m[k] for k in (
                "seconds", "prompt_tokens", "generated_tokens", "all_tokens_per_second", "requests_equal_in_both_runs")},
            "config": {"model": "gpt2-" + args.model, "n_layer": cfg["n_layer"], "n_embd": cfg["n_embd"],
                       "n_head": cfg["n_head"], "requests": m["requests"], "max_chunk": 512, "step_tokens": args.step_tokens, "page_size": args.page_size,
                       "steps": m["steps"], "mean_batch_tokens": m["mean_batch_tokens"], "preemptions": m["preemptions"],
                       "pool_tokens": model.engine_config.max_cached_tokens}}))
        return 0

    with tempfile.TemporaryDirectory() as folder:
        random_model(folder, cfg, seed=0)
        model = engine_from_folder(folder, args.dtype, max(args.batch, 64 if not args.no_points else args.batch), cfg,
                                   kernels=args.kernels, max_batch_tokens=max(2048, args.batch, pf_n * pf_len), page_size=args.page_size)
    dt, ctx_mean = decode_run(model, cfg, rng, args.batch, args.prompt_len, args.steps, args.warmup)
    achieved = decode_roofline(cfg, el, args.batch, ctx_mean, dt / args.steps)
    out = {
        "metric": "decode tok/s (GPT-2 %s layer sizes, batch %d, %d-token prompts)" % (args.model, args.batch, args.prompt_len),
        "value": round(args.batch * args.steps / dt, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(dt / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dkey, "data": "synthetic (random weights, uniform-random token ids)",
        "config": {"model": "gpt2-" + args.model, "n_layer": cfg["n_layer"], "n_layer_full": full_layers,
                   "n_embd": cfg["n_embd"], "n_head": cfg["n_head"], "n_inner": 4 * cfg["n_embd"],
                   "vocab_size": cfg["vocab_size"], "n_positions": cfg["n_positions"],
                   "global_batch": args.batch, "seq_len": int(round(ctx_mean)),
                   "prompt_len": args.prompt_len, "page_size": args.page_size, "kernels": args.kernels, "parallelism": "single-gpu"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4)},
    }
    points, fracs = {}, {}
    if not args.no_points:
        for b in (1, 64):
            steps = min(args.steps, 128)
            d, cm = decode_run(model, cfg, rng, b, args.prompt_len, steps, 8)
            points[f"decode_b{b}"] = round(b * steps / d, 1)
            fracs[f"decode_b{b}"] = round(decode_roofline(cfg, el, b, cm, d / steps) / HBM_GBS, 4)
    if not args.no_prefill:
        out["prefill"] = prefill_run(model, cfg, rng, dkey, pf_n, pf_len)
    if args.profile_stages:
        kernel_table(model, cfg, rng, args.batch, args.prompt_len, pf_n, pf_len)
    del model

    if not args.no_extra and args.dtype == "bfloat16":
        # GPT-2 1.5B layer sizes, all 48 layers: decode at batch 1, 8 and 64 and the prefill of 2,048 tokens
        big = model_config("1.5b")
        model = engine_from_gpu_weights(big, args.dtype, 64, kernels=args.kernels)
        for b in (1, 8, 64):
            steps = min(args.steps, 64)
            d, cm = decode_run(model, big, rng, b, args.prompt_len, steps, 4)
            points[f"gpt2_1p5b_decode_b{b}"] = round(b * steps / d, 1)
            fracs[f"gpt2_1p5b_decode_b{b}"] = round(decode_roofline(big, el, b, cm, d / steps) / HBM_GBS, 4)
        pf = prefill_run(model, big, rng, dkey)
        points["gpt2_1p5b_prefill_2048"] = pf["value"]
        fracs["gpt2_1p5b_prefill_2048"] = pf["frac"]
        del model
        # GPT-2 355M layer sizes: the mixed workload
        mid = model_config("355m")
        model = engine_from_gpu_weights(mid, args.dtype, 64, kernels=args.kernels, max_batch_tokens=512 + 64, max_chunk=512)
        m = mixed_run(model, mid, rng)
        points["gpt2_355m_mixed_generated"] = m["value"]
        points["gpt2_355m_mixed_all_tokens"] = m["all_tokens_per_second"]
        points["gpt2_355m_mixed_requests_equal_in_both_runs"] = m["requests_equal_in_both_runs"]
        fracs["gpt2_355m_mixed_flops"] = round(
            (2 * (m["prompt_tokens"] + m["generated_tokens"]) * (weight_bytes(mid, 1) - mid["vocab_size"] * mid["n_embd"])
             + 2 * m["generated_tokens"] * mid["vocab_size"] * mid["n_embd"]) / m["seconds"] / PEAK_FLOPS[dkey], 4)
        out["config"]["points_gpt2_1p5b"] = "n_layer 48 of 48, n_embd 1600, n_head 25, n_inner 6400, decode after 512-token prompts"
        out["config"]["points_gpt2_355m_mixed"] = ("n_layer 24 of 24, n_embd 1024, n_head 16: %d requests at once, prompts 16..%d, "
                                                   "128 new tokens each, portions of 512 beside decoding, %d steps"
                                                   % (m["requests"], m["longest_prompt"], m["steps"]))
        del model
    if points:
        out["points"] = points
        out["points_frac"] = fracs          # decode: of 8 TB/s; prefill and mixed: of the matrix peak
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
