"""Run-time settings of the engine (not read from config.json).

The reference keeps the like in its builder (core/src/main/java/io/teknek/deliverance/
model/AutoModelForCausaLm.java:106-134: working dtype, ``maxBatchSize`` 512, KV settings)
and in ``AutoModelConfig`` (core/.../model/AutoModelConfig.java:20-33).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

DTYPE_NAMES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "BF16": "bfloat16",
               "float32": "float32", "fp32": "float32", "f32": "float32", "F32": "float32"}


KERNEL_MODES = ("tuned", "reference")
PAGE_SIZES = (16, 32, 64)


def check_page_size(page_size: int) -> int:
    """The page sizes every attention kernel takes (the bfloat16 kernels walk keys in aligned runs of
    64); refused here, before anything is reserved, rather than at the first launch."""
    if page_size not in PAGE_SIZES:
        raise ValueError(f"page_size must be one of {PAGE_SIZES}, found {page_size}")
    return page_size


@dataclass
class EngineConfig:
    dtype: str = "bfloat16"            # "bfloat16" (serving kernels) or "float32" (true 32-bit)
    # "tuned": matrix-core products and the prefill/decode attention kernels in bfloat16; "reference":
    # the plain kernels in bfloat16 too, which splits a mismatch into "tuned kernel" or "bfloat16
    # rounding" (the reference picks its math provider in the same place:
    # core/src/main/java/io/teknek/deliverance/benchmark/InferenceBenchmark.java:1067,1139).
    # 32-bit always runs the plain kernels.
    kernels: str = "tuned"
    page_size: int = 16                # tokens per KV page: 16, 32 or 64 (what every attention kernel takes)
    max_cached_tokens: Optional[int] = None   # pool size in tokens; None: sized from free memory
    max_num_seqs: int = 64             # live requests at a time
    max_batch_tokens: int = 2048       # token budget of one step
    max_chunk: int = 512               # largest prompt portion (the reference's maxBatchSize)
    state_slots: Optional[int] = None  # slots for fixed-size per-request state; None: max_num_seqs
    use_graphs: bool = True            # replay decode-only steps from captured HIP graphs
    run_ahead: bool = True             # launch the next decode step before the running one's tokens are read
    native_step: bool = True           # the layer loop in one call into the library where the parts allow it
    poison_freed_pages: bool = False   # debug: a page that goes back is filled with NaN again
    device: str = "cuda:0"

    def __post_init__(self):
        if self.dtype not in DTYPE_NAMES:
            raise ValueError(f"dtype must be bfloat16 or float32, found {self.dtype!r}")
        self.dtype = DTYPE_NAMES[self.dtype]
        if self.kernels not in KERNEL_MODES:
            raise ValueError(f"kernels must be one of {KERNEL_MODES}, found {self.kernels!r}")
        check_page_size(self.page_size)
        if self.max_num_seqs <= 0 or self.max_batch_tokens <= 0 or self.max_chunk <= 0:
            raise ValueError("max_num_seqs, max_batch_tokens and max_chunk must be positive")
