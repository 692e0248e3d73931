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
from typing import Dict, List, Optional


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


class KernelProfiler:
    """Device time of every kernel launch by name, beside what the launch has to move and to compute.

    While enabled, each kernel face in ``kernels.ops`` brackets its launch with two timing events on
    the launch stream and states the bytes the kernel must read and write at least (every operand
    once) and its floating-point operations; ``summary()`` sets the measured time against the
    MI355X's peaks (8 TB/s of HBM; 2.5 PFLOP/s of bfloat16 matrix products, 157.3 TFLOP/s of
    32-bit arithmetic): the fraction of the roofline that binds that kernel, i.e. the larger of the
    two.  Steps must run kernel by kernel for this (the engine switches recorded graphs off), and
    the events cost a few microseconds a launch: what two events with nothing between them measure
    (the median of 200 pairs, ``overhead_us``) is taken off every launch, and the totals are still for
    comparison between kernels, not the engine's speed.  The reference prints per-stage totals in the same place
    (core/src/main/java/io/teknek/deliverance/model/InferenceProfiler.java:44-82)."""
    enabled = False
    HBM_BYTES_PER_S = 8.0e12
    PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
    _open: List[tuple] = []          # (name, bytes, flops, precision, start event, end event)
    overhead_us: Optional[float] = None   # what a pair of events measures with no kernel between them

    @classmethod
    def enable(cls) -> None:
        cls.enabled = True
        cls._open = []

    @classmethod
    def disable(cls) -> None:
        cls.enabled = False

    @classmethod
    def reset(cls) -> None:
        cls._open = []

    @classmethod
    @contextmanager
    def launch(cls, name: str, nbytes: float, flops: float, precision: str = "bf16"):
        import torch
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        try:
            yield
        finally:
            b.record()
            cls._open.append((name, float(nbytes), float(flops), precision, a, b))

    @classmethod
    def calibrate(cls) -> float:
        import torch
        pairs = []
        for _ in range(200):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record(); b.record()
            pairs.append((a, b))
        torch.cuda.synchronize()
        times = sorted(a.elapsed_time(b) * 1e3 for a, b in pairs)
        cls.overhead_us = times[len(times) // 2]
        return cls.overhead_us

    @classmethod
    def rows(cls) -> List[dict]:
        """One record per kernel name: calls, total microseconds, bytes, flops, GB/s, TFLOP/s and the
        fraction of the binding roofline."""
        import torch
        torch.cuda.synchronize()
        if cls.overhead_us is None:
            cls.calibrate()
        acc: Dict[str, list] = {}
        for name, nb, fl, prec, a, b in cls._open:
            r = acc.setdefault(name, [0, 0.0, 0.0, 0.0, prec])
            r[0] += 1
            r[1] += max(a.elapsed_time(b) * 1e3 - cls.overhead_us, 0.1)        # microseconds
            r[2] += nb
            r[3] += fl
        out = []
        for name, (n, us, nb, fl, prec) in acc.items():
            secs = max(us * 1e-6, 1e-12)
            mem = nb / secs / cls.HBM_BYTES_PER_S
            alu = fl / secs / cls.PEAK_FLOPS[prec]
            out.append(dict(kernel=name, calls=n, total_us=us, mean_us=us / n, gbytes_per_s=nb / secs / 1e9,
                            tflops=fl / secs / 1e12, bound="hbm" if mem >= alu else "flops", frac=max(mem, alu)))
        return sorted(out, key=lambda r: -r["total_us"])

    @classmethod
    def summary(cls, label: str = "") -> str:
        rows = cls.rows()
        total = sum(r["total_us"] for r in rows) or 1.0
        lines = [f"kernel summary {label}".rstrip() + f" ({cls.overhead_us:.1f} us of event overhead taken off every launch)",
                 f"{'kernel':28s} {'calls':>7s} {'total_us':>11s} {'mean_us':>9s} {'%time':>6s} {'GB/s':>9s} {'TFLOP/s':>9s} "
                 f"{'bound':>6s} {'%roofline':>9s}"]
        for r in rows:
            lines.append(f"{r['kernel']:28s} {r['calls']:7d} {r['total_us']:11.1f} {r['mean_us']:9.2f} "
                         f"{100 * r['total_us'] / total:6.1f} {r['gbytes_per_s']:9.1f} {r['tflops']:9.2f} {r['bound']:>6s} "
                         f"{100 * r['frac']:9.2f}")
        return "\n".join(lines)
