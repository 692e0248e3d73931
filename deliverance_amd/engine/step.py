"""The step function: one batch of (request, its next tokens) through the model.

A step may mix portions of prompts with single decoded tokens, cut anywhere.  It runs only
the tokens it is given, against the cache that earlier steps left, and returns the logits at
the wanted places.  The reference has two entry points for one request at a time
(``batchForward`` for a prompt in chunks of 512 and ``forward`` for one token:
core/src/main/java/io/teknek/deliverance/model/AbstractModel.java:1011-1048,1064-1072); both
collapse into this one function, and so does the head that its sampler applies to the last
row (core/.../model/AbstractGeneratorSampler.java:112-115).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import torch

from ..cache.manager import OutOfPages
from ..models.causal_lm import CausalLM
from ..parts.base import Arena, StepContext
from .device_cache import DeviceCache


@dataclass
class StepEntry:
    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=list)    # places among ``tokens`` whose logits are wanted


class StepError(ValueError):
    pass


class StepRunner:
    def __init__(self, model: CausalLM, cache: DeviceCache):
        self.model = model
        self.cache = cache
        self.device = model.device
        self.arena = Arena(self.device)
        self._staging: Optional[torch.Tensor] = None     # pinned host buffer for the step's integers
        self._staging_dev: Optional[torch.Tensor] = None
        self._copied = None
        self.max_blocks_cap = -(-model.config.max_positions // cache.page_size)
        self.last_ctx: Optional[StepContext] = None

    # ---- host -> device in one copy --------------------------------------------------------
    def _upload(self, words: List[int]) -> torch.Tensor:
        n = len(words)
        if self._staging is None or self._staging.numel() < n:
            cap = max(4096, 2 * n)
            self._staging = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._staging_dev = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._copied = None
        if self._copied is not None:
            self._copied.synchronize()       # the last step's copy has read the pinned buffer
        self._staging[:n] = torch.tensor(words, dtype=torch.int32)
        self._staging_dev[:n].copy_(self._staging[:n], non_blocking=True)
        self._copied = torch.cuda.Event()
        self._copied.record()
        return self._staging_dev

    # ---- the step --------------------------------------------------------------------------
    def run(self, entries: Sequence[StepEntry], reserved: bool = False,
            extra_words: Optional[List[int]] = None):
        """Run one step.  Returns (logits [R, V] float32 on the device, ctx).  The rows follow
        the order of ``entries`` and of each entry's ``want``.  With ``reserved`` the caller has
        already opened the requests and reserved their positions (``CacheManager.extend``).
        ``extra_words`` ride along in the same host-to-device copy (``ctx.extra``)."""
        mgr = self.cache.manager
        cfg = self.model.config
        if not entries:
            raise StepError("a step needs at least one entry")
        seen = set()
        for e in entries:
            if e.rid in seen:
                raise StepError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            if len(e.tokens) == 0:
                raise StepError(f"request {e.rid!r} brings no tokens")
            for t in e.tokens:
                if not (0 <= int(t) < cfg.vocab_size):
                    raise StepError(f"request {e.rid!r}: token id {t} is outside the vocabulary of {cfg.vocab_size}")
            for w in e.want:
                if not (0 <= int(w) < len(e.tokens)):
                    raise StepError(f"request {e.rid!r}: wanted place {w} is outside its {len(e.tokens)} tokens")

        starts = {}
        if reserved:
            for e in entries:
                starts[e.rid] = mgr.length(e.rid)
        else:
            done = []
            opened = []
            try:
                for e in entries:
                    if e.rid not in mgr:
                        self.cache.reset_state(mgr.open(e.rid))
                        opened.append(e.rid)
                    if mgr.length(e.rid) + len(e.tokens) > cfg.max_positions:
                        raise StepError(f"request {e.rid!r} would reach position "
                                        f"{mgr.length(e.rid) + len(e.tokens)}, the model has {cfg.max_positions}")
                    starts[e.rid] = mgr.extend(e.rid, len(e.tokens))
                    done.append(e.rid)
            except (OutOfPages, StepError):
                for rid in done:
                    mgr.rollback(rid)
                for rid in opened:
                    mgr.close(rid)
                raise

        # one-token entries first (the decode kernels take them), portions after
        order = sorted(range(len(entries)), key=lambda i: (len(entries[i].tokens) != 1, i))
        n_decode = sum(1 for e in entries if len(e.tokens) == 1)
        S = len(entries)
        tokens: List[int] = []
        positions: List[int] = []
        seq_of: List[int] = []
        q_start = [0]
        seq_lens: List[int] = []
        state_slots: List[int] = []
        row0 = {}
        for s, i in enumerate(order):
            e = entries[i]
            st = starts[e.rid]
            row0[i] = len(tokens)
            tokens += [int(t) for t in e.tokens]
            positions += list(range(st, st + len(e.tokens)))
            seq_of += [s] * len(e.tokens)
            q_start.append(len(tokens))
            seq_lens.append(st + len(e.tokens))
            state_slots.append(mgr.state_slot(e.rid))
        N = len(tokens)
        want_rows = [row0[i] + int(w) for i, e in enumerate(entries) for w in e.want]
        R = len(want_rows)

        G = len(self.cache.groups)
        max_blocks = max(1, max(len(mgr.table(entries[i].rid, g)) for i in order for g in range(G))) if G else 1
        words = tokens + positions + seq_of + q_start + seq_lens + state_slots + want_rows
        offs = {}
        o = 0
        for name, n in (("tokens", N), ("positions", N), ("seq_of", N), ("q_start", S + 1), ("seq_lens", S),
                        ("state_slots", S), ("want", R)):
            offs[name] = (o, n)
            o += n
        for g in range(G):
            sm: List[int] = []
            bt: List[int] = []
            for i in order:
                e = entries[i]
                sm += mgr.slots_for(e.rid, g, starts[e.rid], len(e.tokens))
                t = mgr.table(e.rid, g)
                bt += t + [-1] * (max_blocks - len(t))
            words += sm + bt
            offs[f"slot_map{g}"] = (o, N)
            offs[f"block_table{g}"] = (o + N, S * max_blocks)
            o += N + S * max_blocks
        if extra_words:
            words += extra_words
            offs["extra"] = (o, len(extra_words))
        dev = self._upload(words)

        def view(name):
            a, n = offs[name]
            return dev[a:a + n]

        ctx = StepContext()
        ctx.device = self.device
        ctx.dtype = self.model.dtype
        ctx.n_tokens, ctx.n_seqs, ctx.n_decode = N, S, n_decode
        ctx.tokens, ctx.positions, ctx.seq_of_token = view("tokens"), view("positions"), view("seq_of")
        ctx.q_start, ctx.seq_lens, ctx.state_slots = view("q_start"), view("seq_lens"), view("state_slots")
        ctx.q_start_host, ctx.seq_lens_host, ctx.state_slots_host = q_start, seq_lens, state_slots
        ctx.max_query_len = max(q_start[s + 1] - q_start[s] for s in range(S))
        ctx.max_seq_len = max(seq_lens)
        ctx.block_tables = [view(f"block_table{g}").view(S, max_blocks) for g in range(G)]
        ctx.slot_maps = [view(f"slot_map{g}") for g in range(G)]
        ctx.cache = self.cache
        ctx._arena = self.arena
        ctx.extra = view("extra") if extra_words else None
        self.last_ctx = ctx

        logits = self.model.forward(ctx, view("want") if R else None, R)
        if not reserved:                 # who reserves commits: the scheduler does it for its batches
            for e in entries:
                mgr.commit(e.rid)
        return logits, ctx
