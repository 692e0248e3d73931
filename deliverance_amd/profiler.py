"""Named stage timers, off unless asked for.

The reference keeps a static registry of named timers and counters with exact totals, switched
on by ``--profile-stages`` and printed as a summary (core/src/main/java/io/teknek/deliverance/
model/InferenceProfiler.java:24-161; stage names such as ``generation.prefill``,
``generation.decode``, ``sampler.sample``: core/.../model/GenerationEngine.java:83-146).  Here a
stage is host time around a part of an engine step; with ``sync=True`` the GPU is drained at
each stage's end so that the time is the stage's own (this slows the engine and is for
diagnosis only).  Per-kernel times come from ``rocprofv3``.
"""
from __future__ import annotations

import time
from contextlib import contextmanager
from typing import Dict, List


class InferenceProfiler:
    enabled = False
    sync = False
    _totals: Dict[str, List[float]] = {}

    @classmethod
    def enable(cls, sync: bool = False) -> None:
        cls.enabled, cls.sync = True, sync

    @classmethod
    def reset(cls) -> None:
        cls._totals = {}

    @classmethod
    @contextmanager
    def timer(cls, name: str):
        if not cls.enabled:
            yield
            return
        t0 = time.perf_counter_ns()
        try:
            yield
        finally:
            if cls.sync:
                import torch
                torch.cuda.synchronize()
            rec = cls._totals.setdefault(name, [0, 0])
            rec[0] += 1
            rec[1] += time.perf_counter_ns() - t0

    @classmethod
    def counter(cls, name: str, n: int = 1) -> None:
        if cls.enabled:
            rec = cls._totals.setdefault(name, [0, 0])
            rec[0] += n

    @classmethod
    def summary(cls, label: str = "", max_rows: int = 40) -> str:
        rows = sorted(cls._totals.items(), key=lambda kv: -kv[1][1])[:max_rows]
        lines = [f"profile summary {label}".rstrip(), f"{'stage':40s} {'count':>10s} {'total_ms':>12s} {'mean_us':>10s}"]
        for name, (n, ns) in rows:
            lines.append(f"{name:40s} {n:10d} {ns / 1e6:12.3f} {(ns / n / 1e3 if n else 0):10.1f}")
        return "\n".join(lines)
