"""Command line.  Option names and meanings follow the reference's benchmark main where it has
them (core/src/main/java/io/teknek/deliverance/benchmark/InferenceBenchmark.java:1036-1141):
``--model``, ``--working-dtype``, ``--kernels`` (the reference's ``--tensor-provider``), ``--max-tokens`` (256), ``--temperature`` (0.0), ``--seed N|none``
(42), ``--warmup-cases`` (1), ``--max-cases``, ``--kv-context-rows-per-page``, ``--model-config``,
``--profile-stages``, ``--suite-file``, ``--output`` (CSV), ``--jsonl-output``.  The engine works
on token ids, so prompts are lists of ids (``--prompt-ids 5,17,3`` or a JSONL suite file with a
``prompt_ids`` list per line).  ``--model`` is a local folder; nothing is downloaded.

    python -m deliverance_amd generate --model DIR --prompt-ids 1,2,3 --max-tokens 32
    python -m deliverance_amd random --config config.json --seed 0 --out DIR
    python -m deliverance_amd inspect DIR
"""
from __future__ import annotations

import argparse
import csv
import json
import sys
import time


def _dtype_name(s: str) -> str:
    m = {"BF16": "bfloat16", "F32": "float32", "BFLOAT16": "bfloat16", "FLOAT32": "float32", "FP32": "float32"}
    if s.upper() not in m:
        raise argparse.ArgumentTypeError("working dtype must be BF16 or F32")
    return m[s.upper()]


def _seed(s: str):
    return None if s.lower() == "none" else int(s)


def _ids(s: str):
    return [int(t) for t in s.replace(" ", "").split(",") if t]


def cmd_generate(a) -> int:
    from . import AutoModelForCausalLM, EngineConfig, GeneratorParameters
    from .profiler import InferenceProfiler, KernelProfiler
    prompts = [_ids(p) for p in (a.prompt_ids or [])]
    if a.suite_file:
        with open(a.suite_file) as f:
            for line in f:
                line = line.strip()
                if line:
                    prompts.append([int(t) for t in json.loads(line)["prompt_ids"]])
    if not prompts:
        print("no prompts: give --prompt-ids or --suite-file", file=sys.stderr)
        return 2
    if a.max_cases is not None:
        prompts = prompts[:a.max_cases]
    cfg = {}
    if a.model_config:
        with open(a.model_config) as f:
            cfg = json.load(f)
    cfg.update({k: v for k, v in dict(dtype=a.working_dtype, kernels=a.kernels, page_size=a.kv_context_rows_per_page,
                                      max_batch_tokens=a.max_batch_tokens, max_num_seqs=a.max_num_seqs,
                                      max_cached_tokens=a.max_cached_tokens).items() if v is not None})
    if a.profile_stages:
        InferenceProfiler.enable(sync=True)
        KernelProfiler.enable()            # every kernel launch timed on the device (no recorded graphs meanwhile)
    model = AutoModelForCausalLM.from_pretrained(a.model, engine_config=EngineConfig(**cfg))
    params = GeneratorParameters(temperature=a.temperature, seed=a.seed, max_tokens=a.max_tokens, ntokens=a.ntokens,
                                 top_k=a.top_k, top_p=a.top_p, uniform_top_p=a.uniform_top_p,
                                 xtc_threshold=a.xtc_threshold, xtc_probability=a.xtc_probability,
                                 ignore_eos=a.ignore_eos)
    for p in prompts[:a.warmup_cases]:
        model.generate(p, params)
    InferenceProfiler.reset()
    KernelProfiler.reset()
    t0 = time.perf_counter()
    outs = model.generate(prompts, params) if a.batch else [model.generate(p, params) for p in prompts]
    wall = time.perf_counter() - t0
    rows = []
    for p, r in zip(prompts, outs):
        n = len(r.generated_tokens)
        decode_ms = max(0.0, r.total_time_ms - r.time_to_first_token_ms)
        # the reference's request line (core/.../model/GenerationEngine.java:259-266)
        print(f"generation_complete prompt_tokens={r.prompt_tokens} generated_tokens={n} total_ms={r.total_time_ms:.3f} "
              f"ttft_ms={r.time_to_first_token_ms:.3f} tokens_per_second={n * 1e3 / r.total_time_ms if r.total_time_ms else 0:.3f} "
              f"decode_tokens_per_second={(n - 1) * 1e3 / decode_ms if decode_ms > 0 and n > 1 else 0:.3f} "
              f"finish_reason={r.finish_reason}", file=sys.stderr)
        print(",".join(str(t) for t in r.generated_tokens))
        rows.append(dict(prompt_tokens=r.prompt_tokens, generated_tokens=n, total_ms=round(r.total_time_ms, 3),
                         generation_ms=round(decode_ms, 3),
                         tokens_per_second=round(n * 1e3 / r.total_time_ms, 3) if r.total_time_ms else 0,
                         finish_reason=r.finish_reason, token_ids=r.generated_tokens, prompt_ids=p))
    total = sum(r["generated_tokens"] for r in rows)
    print(f"requests={len(rows)} generated_tokens={total} wall_s={wall:.3f} tokens_per_second={total / wall:.1f}", file=sys.stderr)
    if a.output:
        with open(a.output, "w", newline="") as f:
            w = csv.writer(f)
            w.writerow(["prompt_tokens", "generated_tokens", "total_ms", "generation_ms", "tokens_per_second"])
            for r in rows:
                w.writerow([r[k] for k in ("prompt_tokens", "generated_tokens", "total_ms", "generation_ms", "tokens_per_second")])
    if a.jsonl_output:
        with open(a.jsonl_output, "w") as f:
            for r in rows:
                f.write(json.dumps(r) + "\n")
    if a.profile_stages:
        print(InferenceProfiler.summary("(stages drained at their end)"), file=sys.stderr)
        print(KernelProfiler.summary("(device time per kernel against what it must move and compute; % of 8 TB/s or of "
                                     "the matrix peak, whichever binds)"), file=sys.stderr)
    return 0


def cmd_random(a) -> int:
    from .random_model import random_model
    with open(a.config) as f:
        cfg = json.load(f)
    print(random_model(a.out, cfg, a.seed))
    return 0


def cmd_inspect(a) -> int:
    """Tensor names, dtypes and shapes of a model folder (the reference has
    safetensors/src/main/java/io/teknek/deliverance/safetensors/ModelInspectionMain.java)."""
    from .registry import ModelSupport, read_config_json
    from .weights import WeightSource
    from . import models  # noqa: F401
    cfg = read_config_json(a.model)
    arch = ModelSupport.detect(cfg)
    mc = arch.read_config(cfg)
    print(f"architecture {arch.name}: {len(mc.layers)} layers, width {mc.width}, vocabulary {mc.vocab_size}, "
          f"{mc.max_positions} positions, {len(mc.schedule)} layer calls, {mc.n_cache_slots} cache slots")
    src = WeightSource(a.model)
    total = 0
    for n in sorted(src.names()):
        dt, shape = src.info(n)
        k = 1
        for d in shape:
            k *= d
        total += k
        print(f"{n:50s} {dt:5s} {list(shape)}")
    print(f"{total} parameters in {len(src.names())} tensors")
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="deliverance_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    g = sub.add_parser("generate", help="generate tokens for prompts of token ids")
    g.add_argument("--model", required=True, help="model folder (config.json + safetensors)")
    g.add_argument("--working-dtype", type=_dtype_name, default=None, help="BF16 (default) or F32")
    g.add_argument("--kernels", choices=["tuned", "reference"], default=None,
                   help="bfloat16: the serving kernels (default) or the plain kernels, as the reference's "
                        "--tensor-provider picks its math")
    g.add_argument("--prompt-ids", action="append", help="comma-separated token ids; may be given several times")
    g.add_argument("--suite-file", help="JSONL, one object with a prompt_ids list per line")
    g.add_argument("--max-tokens", type=int, default=256, help="max generated tokens per prompt, default 256")
    g.add_argument("--ntokens", type=int, default=None, help="bound on prompt + generated positions")
    g.add_argument("--temperature", type=float, default=0.0, help="default 0.0 (greedy)")
    g.add_argument("--seed", type=_seed, default=42, help="N or none, default 42")
    g.add_argument("--top-k", type=float, default=None)
    g.add_argument("--top-p", type=float, default=None)
    g.add_argument("--uniform-top-p", type=float, default=None)
    g.add_argument("--xtc-threshold", type=float, default=None)
    g.add_argument("--xtc-probability", type=float, default=None)
    g.add_argument("--ignore-eos", action="store_true")
    g.add_argument("--warmup-cases", type=int, default=1, help="prompts to run before recording, default 1")
    g.add_argument("--max-cases", type=int, default=None)
    g.add_argument("--kv-context-rows-per-page", type=int, default=None, help="tokens per cache page, default 16")
    g.add_argument("--max-batch-tokens", type=int, default=None)
    g.add_argument("--max-num-seqs", type=int, default=None)
    g.add_argument("--max-cached-tokens", type=int, default=None)
    g.add_argument("--model-config", help="JSON file with engine settings (EngineConfig fields)")
    g.add_argument("--no-batch", dest="batch", action="store_false", help="one request at a time, as the reference runs them")
    g.add_argument("--profile-stages", action="store_true")
    g.add_argument("--output", help="CSV: prompt_tokens,generated_tokens,total_ms,generation_ms,tokens_per_second")
    g.add_argument("--jsonl-output")
    g.set_defaults(fn=cmd_generate)
    r = sub.add_parser("random", help="write a model folder with seeded random weights")
    r.add_argument("--config", required=True)
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--out", required=True)
    r.set_defaults(fn=cmd_random)
    i = sub.add_parser("inspect", help="list a model folder's tensors")
    i.add_argument("model")
    i.set_defaults(fn=cmd_inspect)
    a = ap.parse_args(argv)
    return a.fn(a)


if __name__ == "__main__":
    sys.exit(main())
