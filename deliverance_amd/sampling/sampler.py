"""Host side of sampling: the per-request random stream and the records the device kernel
reads.  The pick itself runs on the GPU (csrc/sample.hip).

The reference seeds a ``java.util.Random`` per request (core/src/main/java/io/teknek/
deliverance/model/GenerationEngine.java:89) and draws from it once when a sampler is made
for a token (core/.../model/AbstractModel.java:826,836), once per "exclude top choices"
picker (core/.../model/ExcludeTopChoicePicker.java:43) and once for the pick
(core/.../model/AbstractGeneratorSampler.java:211).  The same generator and the same order
of draws are kept here, so a request's tokens depend on its seed and its own logits only,
never on what else is in the batch.
"""
from __future__ import annotations

import math
import struct
from typing import Optional

from .params import GeneratorParameters

RECORD_WORDS = 8      # one device record: 8 four-byte fields (see SampleRow in csrc/sample.hip)


class JavaRandom:
    """The 48-bit linear congruential generator of java.util.Random."""
    _MASK = (1 << 48) - 1

    def __init__(self, seed: Optional[int]):
        if seed is None:
            import os
            seed = int.from_bytes(os.urandom(6), "little")
        self._s = (int(seed) ^ 0x5DEECE66D) & self._MASK

    def _next(self, bits: int) -> int:
        self._s = (self._s * 0x5DEECE66D + 0xB) & self._MASK
        return self._s >> (48 - bits)

    def next_float(self) -> float:
        return self._next(24) / float(1 << 24)


def top_k_candidate_count(top_k: float, vocab: int) -> int:
    """Below 1: keep ``max(1, V - int(k V))``; from 1 up: ``min(V, round(k))``
    (AbstractGeneratorSampler.java:256-264)."""
    if top_k <= 0:
        raise ValueError("topK must be > 0")
    if top_k < 1.0:
        f = struct.unpack("f", struct.pack("f", top_k))[0]
        prod = struct.unpack("f", struct.pack("f", f * float(vocab)))[0]
        return max(1, vocab - int(prod))
    return min(vocab, int(math.floor(top_k + 0.5)))


def device_record(p: GeneratorParameters, rng: JavaRandom, vocab: int) -> bytes:
    """Advance the request's random stream for one token and pack the kernel's record."""
    rng.next_float()                                   # drawn when the sampler is made; unused
    xtc_on = p.xtc_threshold is not None and p.xtc_threshold != 0.0
    xtc_active = 0
    u = 0.0
    if xtc_on:
        prob = p.xtc_probability or 0.0
        draw = rng.next_float()                        # picker on the raw logits
        if p.temperature == 0.0:
            xtc_active = int(not (draw > prob))
        else:
            draw = rng.next_float()                    # second picker, on logits / temperature
            xtc_active = int(not (draw > prob))
    elif p.temperature > 0.0:
        u = rng.next_float()
    top_k = 0 if p.top_k is None else top_k_candidate_count(p.top_k, vocab)
    return struct.pack("<fififfii", float(p.temperature), int(top_k), float(p.top_p or 0.0),
                       int(p.uniform_top_p is not None), float(u),
                       float(p.xtc_threshold) if xtc_on else 0.0, int(xtc_active), 0)


def greedy_record() -> bytes:
    return struct.pack("<fififfii", 0.0, 0, 0.0, 0, 0.0, 0.0, 0, 0)
