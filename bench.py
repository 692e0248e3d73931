#!/usr/bin/env python3
"""Serving benchmark on one MI355X: decode tokens a second at a fixed batch, prefill of 2,048
tokens, and the decode step's fraction of the HBM roofline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--model 124m|355m|1.5b] [--batch B]

A "step" is one decode step of the engine (scheduler decision, model step over the paged cache,
sampling on the device, tokens back on the host).  Weights are random (N(0, 0.02)), prompts are
seeded uniform-random token ids of 512 tokens, decoding is greedy and ignores end tokens.
Prints ONE JSON line.
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


def model_config(name, n_layer=None):
    c = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", vocab_size=50257, n_positions=1024,
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


def mixed_run(args, cfg, folder, rng, dkey):
    """Continuous batching under load: every request arrives at once; the scheduler admits them as
    seats and pages allow, cuts prompts into portions of at most 512 tokens and runs them in the
    same steps as the other requests' decoding.  One JSON line: generated tokens a second over the
    whole run (prompt processing included)."""
    import torch
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    n_req, new = 64, 128
    longest = cfg["n_positions"] - new - 1
    model = AutoModelForCausalLM.from_pretrained(
        folder, dtype=args.dtype, max_num_seqs=n_req, max_batch_tokens=512 + n_req, max_chunk=512,
        max_cached_tokens=n_req * cfg["n_positions"], page_size=16)
    lengths = [int(x) for x in rng.integers(16, longest + 1, size=n_req)]
    prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lengths]
    params = GeneratorParameters(max_tokens=new, ignore_eos=True)
    best = None
    for _ in range(2):                        # the first run records the decode graphs
        before = model.stats()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        outs = model.generate(prompts, params)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if best is None or dt < best:
            best = dt
            after = model.stats()
            steps = after["steps"] - before["steps"]
            batch_tokens = after["batch_tokens"] - before["batch_tokens"]
    assert all(len(o.generated_tokens) == new for o in outs)
    stats = model.stats()
    print(json.dumps({
        "metric": "generated tok/s, %d requests at once (GPT-2 %s layer sizes, prompts 16..%d, %d new tokens each, "
                  "prompt portions of 512 beside decoding)" % (n_req, args.model, longest, new),
        "value": round(n_req * new / best, 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
        "dtype": dkey, "data": "synthetic (random weights, uniform-random token ids)",
        "seconds": round(best, 4), "prompt_tokens": sum(lengths), "generated_tokens": n_req * new,
        "all_tokens_per_second": round((sum(lengths) + n_req * new) / best, 1),
        "config": {"model": "gpt2-" + args.model, "n_layer": cfg["n_layer"], "n_embd": cfg["n_embd"],
                   "n_head": cfg["n_head"], "requests": n_req, "max_chunk": 512, "page_size": 16,
                   "steps": steps, "mean_batch_tokens": round(batch_tokens / max(steps, 1), 1),
                   "preemptions": stats.get("preemptions", 0)}}))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="124m", choices=sorted(MODELS))
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed"],
                    help="mixed: 64 requests with prompts of 16 to 895 tokens arrive at once, prompt portions of 512 "
                         "tokens run beside the decoding of the others, 128 new tokens each (use --model 355m)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    import numpy as np
    import torch
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    from deliverance_amd.random_model import random_model

    cfg = model_config(args.model, args.layers)
    full_layers = MODELS[args.model]["n_layer"]
    el = 2 if args.dtype == "bfloat16" else 4
    dkey = "bf16" if args.dtype == "bfloat16" else "fp32"
    rng = np.random.default_rng(0)

    def prompts(n, length):
        return [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=length)] for _ in range(n)]

    with tempfile.TemporaryDirectory() as folder:
        random_model(folder, cfg, seed=0)
        total_new = args.steps + args.warmup + 1
        if args.prompt_len + total_new > cfg["n_positions"]:
            print(f"prompt {args.prompt_len} + {total_new} decoded tokens exceed n_positions {cfg['n_positions']}")
            return 2

        def engine(batch):
            return AutoModelForCausalLM.from_pretrained(
                folder, dtype=args.dtype, max_num_seqs=max(batch, 2), max_batch_tokens=max(2048, batch),
                max_chunk=1024, max_cached_tokens=max(batch, 2) * cfg["n_positions"], page_size=16)

        def decode_run(model, batch, steps, warmup):
            """Prefill `batch` prompts (untimed), `warmup` decode steps, then time `steps` decode steps."""
            params = GeneratorParameters(max_tokens=steps + warmup + 1, ignore_eos=True)
            for p in prompts(batch, args.prompt_len):
                model.add_request(p, params)
            while any(r.n_computed < len(r.prompt) for r in model.scheduler.running) or model.scheduler.waiting:
                model.step()
            for _ in range(warmup):
                model.step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                model.step()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            ctx_mean = args.prompt_len + 1 + warmup + steps / 2.0
            while model.has_work():
                model.step()
            model.scheduler.finished.clear()
            return dt, ctx_mean

        if args.workload == "mixed":
            return mixed_run(args, cfg, folder, rng, dkey)
        model = engine(max(args.batch, 64 if not args.no_points else args.batch))
        dt, ctx_mean = decode_run(model, args.batch, args.steps, args.warmup)
        ms_per_step = dt / args.steps * 1e3
        value = args.batch * args.steps / dt
        kv_bytes_per_token = 2 * cfg["n_embd"] * el * cfg["n_layer"]
        step_bytes = weight_bytes(cfg, el) + args.batch * ctx_mean * kv_bytes_per_token
        achieved = step_bytes / (dt / args.steps) / 1e9
        out = {
            "metric": "decode tok/s (GPT-2 %s layer sizes, batch %d, 512-token prompts)" % (args.model, args.batch),
            "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": dkey, "data": "synthetic (random weights, uniform-random token ids)",
            "config": {"model": "gpt2-" + args.model, "n_layer": cfg["n_layer"], "n_layer_full": full_layers,
                       "n_embd": cfg["n_embd"], "n_head": cfg["n_head"], "n_inner": 4 * cfg["n_embd"],
                       "vocab_size": cfg["vocab_size"], "n_positions": cfg["n_positions"],
                       "global_batch": args.batch, "seq_len": args.prompt_len + args.warmup + args.steps + 1,
                       "prompt_len": args.prompt_len, "page_size": 16, "parallelism": "single-gpu"},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_GBS, 4)},
        }

        if not args.no_points:
            points = {}
            for b in (1, 64):
                steps = min(args.steps, 128)
                d, _ = decode_run(model, b, steps, 8)
                points[f"decode_b{b}"] = round(b * steps / d, 1)
            out["points"] = points

        if not args.no_prefill:
            # 2 x 1,024-token prompts in ONE step of the engine's step function, logits at the two last rows
            from deliverance_amd.engine.step import StepEntry
            times = []
            for it in range(5):                       # the first rounds warm up; the best of the rest counts
                entries = [StepEntry(f"prefill{i}", p, [len(p) - 1]) for i, p in enumerate(prompts(2, 1024))]
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                logits, _ = model.runner.run(entries)
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
                for e in entries:
                    model.cache.manager.close(e.rid)
            t = min(times[2:])
            ntok = 2 * 1024
            fl = step_flops(cfg, [1024, 1024])
            out["prefill"] = {"value": round(ntok / t, 1), "tokens": ntok, "ms": round(t * 1e3, 3),
                              "frac": round(fl / t / PEAK_FLOPS[dkey], 4)}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
