"""Interfaces of the parts a block is made of, their registries, and the step context.

A part is built from its spec record (sizes and constants as parameters) and a dict of
parameter tensors under the part's own local names; it never sees the model's config or the
checkpoint's tensor names.  Kinds are looked up by ``spec.kind`` in the registries below, so
a new mixer, feed-forward, norm or position encoding is added by registering a builder.

Interfaces (shapes: N tokens of the step, E model width):

* ``Norm.forward(ctx, x, rows=None, out_dtype=None) -> h``: x is the 32-bit residual stream [N, E];
  h is in the compute dtype (or ``out_dtype``), [N, E] or, with ``rows`` (int32 row indices),
  [len(rows), E].
* ``Mixer.forward(ctx, h, x, call) -> None``: reads h, *adds* its result to x in place
  (32-bit).  ``call`` is the run-order entry (cache slot, write flag).
  ``Mixer.cache_need()`` says what the mixer keeps between steps: a ``KVNeed`` (pages of keys
  and values), a ``StateNeed`` (fixed-size state in a slot per request) or None.  A mixer with
  state finds everything about the step's rows on the device (``ctx.seq_of_token``,
  ``ctx.positions``, ``ctx.q_start``, ``ctx.state_slots``); ``ops.state_gather`` hands every row
  its sequence's state and ``ops.state_scatter`` keeps the state that each portion's last row
  leaves.  One that reads these only (never the ``*_host`` lists) may set ``graph_safe``.
* ``FeedForward.forward(ctx, h, x) -> None``: reads h, adds its result to x in place.
* ``PositionEncoding``: ``embed_table()`` returns a [P, E] table added to token embeddings
  (or None); ``apply_qk(ctx, qkv, ...)`` may rotate queries and keys in place (default: none).

The reference wires the same roles through constructor arguments of one block class
(core/src/main/java/io/teknek/deliverance/generator/TransformerBlock.java:26-41,161-200).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Tuple

import torch


@dataclass(frozen=True)
class KVNeed:
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size state of one request: ``elems`` entries of ``dtype``, as one row, or in ``shape`` (whose
    product is ``elems``).  The cache keeps a tensor ``[state slots, *shape]`` of that dtype for it and
    counts its bytes in the memory it plans with."""
    elems: int
    dtype: torch.dtype = torch.float32
    shape: Optional[Tuple[int, ...]] = None

    def __post_init__(self):
        if self.elems <= 0:
            raise ValueError(f"a state of {self.elems} entries")
        if self.shape is not None:
            n = 1
            for d in self.shape:
                n *= int(d)
            if n != self.elems:
                raise ValueError(f"state shape {tuple(self.shape)} does not hold {self.elems} entries")

    @property
    def row_shape(self) -> Tuple[int, ...]:
        return tuple(self.shape) if self.shape is not None else (self.elems,)

    @property
    def nbytes(self) -> int:
        return self.elems * torch.empty((), dtype=self.dtype).element_size()


class StepContext:
    """Everything a part may read about the running step.

    Rows are ordered sequence by sequence; the first ``n_decode`` sequences bring one token
    each, the others bring portions of two or more.
    """

    def __init__(self):
        self.device = None
        self.dtype: torch.dtype = torch.bfloat16       # compute dtype of activations
        self.n_tokens = 0
        self.n_seqs = 0
        self.n_decode = 0                              # leading one-token sequences
        self.tokens: torch.Tensor = None               # int32 [N]
        self.positions: torch.Tensor = None            # int32 [N] position in its own sequence
        self.seq_of_token: torch.Tensor = None         # int32 [N]
        self.q_start: torch.Tensor = None              # int32 [S+1] first row of each sequence
        self.seq_lens: torch.Tensor = None             # int32 [S] length after this step
        self.state_slots: torch.Tensor = None          # int32 [S]
        self.q_start_host: List[int] = []
        self.seq_lens_host: List[int] = []
        self.state_slots_host: List[int] = []
        self.max_query_len = 0
        self.max_seq_len = 0
        self.block_tables: List[torch.Tensor] = []     # per group int32 [S, max_blocks]
        self.slot_maps: List[torch.Tensor] = []        # per group int32 [N]
        self.cache = None                              # engine.DeviceCache
        self._arena = None
        # Called as hook(layer, stage, tensor) with copies of named intermediates (layer -1: the
        # embedding), when set: core/src/main/java/io/teknek/deliverance/model/AbstractModel.java:122-128,505-515.
        self.debug_hook: Optional[Callable] = None

    def buf(self, name: str, rows: int, cols: int, dtype: torch.dtype) -> torch.Tensor:
        """A scratch matrix [rows, cols] that lives until the step ends."""
        return self._arena.get(name, rows, cols, dtype)

    def group_of(self, cache_slot: int) -> int:
        return self.cache.group_of_slot[cache_slot]

    def emit(self, layer: int, stage: str, tensor: torch.Tensor) -> None:
        """Hand a named intermediate of this step to the debug hook, if there is one."""
        if self.debug_hook is not None:
            self.debug_hook(layer, stage, tensor.detach().clone())


class Arena:
    """Named scratch buffers reused from step to step (no allocation in steady state)."""

    def __init__(self, device):
        self.device = device
        self._bufs: Dict[tuple, torch.Tensor] = {}

    def get(self, name, rows, cols, dtype):
        key = (name, cols, dtype)
        t = self._bufs.get(key)
        if t is None or t.shape[0] < rows:
            cap = max(rows, 16) if t is None else max(rows, 2 * t.shape[0])
            t = torch.empty((cap, cols), dtype=dtype, device=self.device)
            self._bufs[key] = t
        return t[:rows]


class Norm:
    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None, out_name: str = "norm",
                out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        raise NotImplementedError

    def fusable_params(self):
        """(gain, bias or None, eps) when this norm is a LayerNorm that a product kernel can apply to
        its own rows (``ops.linear_ln``); None when the norm must run as a kernel of its own."""
        return None


class Mixer:
    # True when `forward` launches the same kernels with the same arguments for every step of one
    # shape and reads the step's data from device memory only: then a decode step can be recorded
    # once as a HIP graph and replayed.  A mixer that reads ctx.*_host must leave this False.
    graph_safe = False

    def cache_need(self):
        return None

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        raise NotImplementedError


class FeedForward:
    graph_safe = False

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        raise NotImplementedError


class PositionEncoding:
    def embed_table(self) -> Optional[torch.Tensor]:
        return None

    def apply_qk(self, ctx: StepContext, qkv: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int) -> None:
        return None


# ---- registries -------------------------------------------------------------------------
# builder(spec, params: dict[str, Tensor], dtype: torch.dtype, device) -> part
_NORMS: Dict[str, Callable] = {}
_MIXERS: Dict[str, Callable] = {}
_FEED_FORWARDS: Dict[str, Callable] = {}
_POSITIONS: Dict[str, Callable] = {}


def _register(table, what):
    def reg(kind: str, builder: Callable, replace: bool = False):
        if kind in table and not replace:
            raise ValueError(f"{what} kind {kind!r} is already registered")
        table[kind] = builder
    return reg


def _build(table, what):
    def build(spec, params, dtype, device):
        kind = getattr(spec, "kind", None)
        if kind not in table:
            raise KeyError(f"no {what} of kind {kind!r}; registered: {sorted(table)}")
        return table[kind](spec, params, dtype, device)
    return build


register_norm = _register(_NORMS, "norm")
register_mixer = _register(_MIXERS, "mixer")
register_feed_forward = _register(_FEED_FORWARDS, "feed-forward")
register_position = _register(_POSITIONS, "position encoding")
build_norm = _build(_NORMS, "norm")
build_mixer = _build(_MIXERS, "mixer")
build_feed_forward = _build(_FEED_FORWARDS, "feed-forward")
build_position = _build(_POSITIONS, "position encoding")


def _owned(out: torch.Tensor, src: torch.Tensor) -> torch.Tensor:
    """A part owns its parameters: when the conversion was a no-op, ``out`` still is the caller's
    memory (a mapped checkpoint file, read-only and at any alignment, or a tensor the caller may
    change), so it is copied."""
    return out.clone() if out.data_ptr() == src.data_ptr() else out


def to_matrix(t: torch.Tensor, dtype: torch.dtype, device) -> torch.Tensor:
    """A matrix operand of the compute dtype on the device ([out, in], contiguous)."""
    return _owned(t.to(device=device, dtype=dtype).contiguous(), t)


def to_vector(t: Optional[torch.Tensor], dtype: torch.dtype, device) -> Optional[torch.Tensor]:
    """A parameter vector: kept in its stored dtype in bfloat16 serving, 32-bit in the 32-bit path."""
    if t is None:
        return None
    if dtype == torch.float32:
        return _owned(t.to(device=device, dtype=torch.float32).contiguous(), t)
    src = t
    if t.dtype not in (torch.bfloat16, torch.float32):
        t = t.to(torch.float32)
    return _owned(t.to(device=device).contiguous(), src)
