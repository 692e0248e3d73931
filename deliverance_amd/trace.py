"""Trace replay: feed given token ids through a model step by step and write logits.

It samples nothing and decides nothing: every step of the trace becomes one call of the
engine's own step function, on the engine's own model, cache manager and kernels.  The
nearest thing in the reference is a test helper that compares cached decoding with a cold
replay (core/src/test/java/io/teknek/deliverance/model/hf/HfGenerationTesterMixinPort.java:16-36).

Input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``<out>/<step>.f32`` holds the logits at the wanted
places, in the order of the entries and of ``want``, as little-endian float32 [wanted, vocab].
After every step a line ``done <step>`` is printed and flushed.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


class TraceSession:
    """The engine's model, cache and step function, driven one trace step at a time.

    ``kernels`` is ``EngineConfig.kernels``.  With ``sample`` every step whose entries all bring one
    token and want its logits runs as generation runs a decode step: greedy sampling records ride
    along, and with ``use_graphs`` the step is padded to a bucket and replayed from a recorded HIP
    graph; ``last_sampled`` then holds the tokens that the device picked."""

    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: int = 16, device: str = "cuda:0",
                 poison_freed: bool = False, kernels: str = "tuned", use_graphs: bool = False, sample: bool = False,
                 native_step: bool = True):
        import torch
        from . import models  # noqa: F401  (registers the architectures)
        from .config.engine_config import KERNEL_MODES
        from .engine.device_cache import DeviceCache
        from .models.causal_lm import load_model
        if kernels not in KERNEL_MODES:
            raise ValueError(f"kernels must be one of {KERNEL_MODES}")
        tdtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
        self.model = load_model(model_dir, tdtype, device)
        # A request's count is rounded up to a multiple of 64, so max_tokens / page_size pages
        # hold every live request whatever its length.
        self.cache = DeviceCache(self.model.cache_needs(), tdtype, device, page_size, max(max_tokens, 64),
                                 n_state_slots=8, poison_freed=poison_freed)
        self.native_step = native_step
        self.runner = self._make_runner(use_graphs, kernels)
        self.sample = sample or use_graphs
        self.last_sampled = None

    def _make_runner(self, use_graphs: bool, kernels: str):
        from .engine.step import StepRunner
        return StepRunner(self.model, self.cache, use_graphs=use_graphs, kernels=kernels, native_step=self.native_step)

    def _drain(self):
        import torch
        torch.cuda.synchronize()

    def run_step(self, rec: dict):
        """One line of the trace.  Returns the wanted logits as a float32 array [wanted, vocab],
        or None when nothing was wanted."""
        import struct
        import torch
        from .engine.step import StepEntry
        from .sampling.params import GeneratorParameters
        from .sampling.sampler import RECORD_WORDS, JavaRandom, device_record
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        out = None
        self.last_sampled = None
        if entries:
            records = None
            if self.sample and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
                one = struct.unpack(f"<{RECORD_WORDS}i", device_record(GeneratorParameters(temperature=0.0), JavaRandom(0),
                                                                       self.model.config.vocab_size))
                records = list(one) * len(entries)
            logits, ctx = self.runner.run(entries, sample_records=records)
            if records is not None:
                picked = getattr(ctx, "sampled", None)
                if picked is None:                      # not replayed from a graph: sample as generation does
                    from .kernels import ops
                    picked = ops.sample(logits, ctx.extra, self.runner.sampled[:len(entries)])
                self.last_sampled = picked.cpu().tolist()
            if logits.shape[0]:
                out = logits.detach().to("cpu", torch.float32).contiguous().numpy()
            else:
                self._drain()
        for rid in rec.get("end", []):
            self.cache.manager.close(rid)
        return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page: 16, 32 or 64")
    ap.add_argument("--kernels", choices=["tuned", "reference"], default="tuned",
                    help="bfloat16 only: the serving kernels (default) or the plain kernels")
    args = ap.parse_args(argv)

    def say(msg):
        print(f"[trace_run] {msg}", file=sys.stderr, flush=True)

    say("importing torch")
    import torch
    from .kernels import build
    if build.library_path() is None:
        say("compiling the HIP kernels (first call)")
    build.load()
    if not torch.cuda.is_available():
        say("no GPU is visible; trace_run drives the GPU engine and has no other path")
        return 3
    say(f"loading {args.model} as {args.dtype}")
    session = TraceSession(args.model, args.dtype, args.max_tokens, args.page_size, kernels=args.kernels)
    os.makedirs(args.out, exist_ok=True)
    say("ready")
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        logits = session.run_step(rec)
        if logits is not None:
            logits.astype("<f4").tofile(os.path.join(args.out, f"{rec['step']}.f32"))
        print(f"done {rec['step']}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
