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
    # The entry's one token is not known on the host yet: it is row ``from_sampled`` of the tokens
    # that the step before sampled on the device (``StepRunner.sampled``); ``tokens`` holds a placeholder.
    from_sampled: Optional[int] = None


class StepError(ValueError):
    pass


class StepRunner:
    def __init__(self, model: CausalLM, cache: DeviceCache, use_graphs: bool = False, max_graph_batch: int = 256):
        self.model = model
        self.cache = cache
        self.device = model.device
        self.arena = Arena(self.device)
        self._staging: Optional[torch.Tensor] = None     # pinned host buffer for the step's integers
        self._staging_dev: Optional[torch.Tensor] = None
        self._copied = None
        self.max_blocks_cap = -(-model.config.max_positions // cache.page_size)
        self.last_ctx: Optional[StepContext] = None
        self.use_graphs = use_graphs and model.graph_safe
        self.max_graph_batch = max_graph_batch
        self._graphs = {}
        # where every sampling step leaves its tokens (row i: the i-th wanted row), and where a step
        # launched on top of it takes them from
        self.sampled = torch.zeros(2 * max(64, max_graph_batch), dtype=torch.int32, device=self.device)

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
            sample_records: Optional[List[int]] = None):
        """Run one step.  Returns (logits [R, V] float32 on the device, ctx).  The rows follow
        the order of ``entries`` and of each entry's ``want``.  With ``reserved`` the caller has
        already opened the requests and reserved their positions (``CacheManager.extend``).
        ``sample_records`` (8 words per wanted row, see sampling.device_record) ride along in the
        same host-to-device copy (``ctx.extra``); when they are given and the step holds one-token
        sequences only, the step and its sampling are replayed from a recorded HIP graph and the
        sampled tokens are left in ``ctx.sampled`` (the first rows of ``self.sampled``)."""
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
            if e.from_sampled is not None and not (len(e.tokens) == 1 and 0 <= e.from_sampled < self.sampled.numel()):
                raise StepError(f"request {e.rid!r}: only a single token can come from the sampled tokens")

        starts = {}
        if reserved:
            for e in entries:               # the entry's tokens are the last positions that were reserved
                starts[e.rid] = mgr.length(e.rid) + mgr.pending(e.rid) - len(e.tokens)
                if starts[e.rid] < mgr.length(e.rid):
                    raise StepError(f"request {e.rid!r} brings {len(e.tokens)} tokens, {mgr.pending(e.rid)} are reserved")
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
        graph_ok = (sample_records is not None and n_decode == len(entries) and self.use_graphs
                    and len(entries) <= self.max_graph_batch and all(list(e.want) == [0] for e in entries))
        if graph_ok:
            logits, ctx = self._run_graph(entries, starts, sample_records)
            if not reserved:
                for e in entries:
                    mgr.commit(e.rid)
            return logits, ctx

        words, offs, meta = self._pack(entries, order, starts, pad_to=None, max_blocks=None,
                                       extra=sample_records)
        dev = self._upload(words)
        ctx = self._context(dev, offs, meta, self.arena)
        self.last_ctx = ctx
        R = meta["R"]
        if any(e.from_sampled is not None for e in entries):
            from ..kernels import ops
            ops.take_tokens(ctx.tokens, ctx.token_src, self.sampled, cfg.vocab_size)
        logits = self.model.forward(ctx, ctx.want_rows if R else None, R)
        if not reserved:                 # who reserves commits: the scheduler does it for its batches
            for e in entries:
                mgr.commit(e.rid)
        return logits, ctx

    # ---- packing the step's integers -----------------------------------------------------------
    def _pack(self, entries, order, starts, pad_to, max_blocks, extra):
        """All integers of a step in one list: tokens, positions, sequence ids, row starts, lengths,
        state slots, wanted rows, then per cache group the cache row of every token and the block
        tables, then ``extra``.  With ``pad_to`` the step is filled up with empty one-token
        sequences (length 0, no cache row), so that its shape is fixed."""
        mgr = self.cache.manager
        S_real = len(entries)
        tokens: List[int] = []
        token_src: List[int] = []
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
            token_src += [e.from_sampled] if e.from_sampled is not None else [-1] * len(e.tokens)
            positions += list(range(st, st + len(e.tokens)))
            seq_of += [s] * len(e.tokens)
            q_start.append(len(tokens))
            seq_lens.append(st + len(e.tokens))
            state_slots.append(mgr.state_slot(e.rid))
        want_rows = [row0[i] + int(w) for i, e in enumerate(entries) for w in e.want]
        n_pad = 0 if pad_to is None else pad_to - S_real
        for k in range(n_pad):
            tokens.append(0); token_src.append(-1); positions.append(0); seq_of.append(S_real + k)
            q_start.append(len(tokens)); seq_lens.append(0); state_slots.append(-1)
            want_rows.append(len(tokens) - 1)
        N, S, R = len(tokens), S_real + n_pad, len(want_rows)
        G = len(self.cache.groups)
        if max_blocks is None:
            max_blocks = max(1, max(len(mgr.table(entries[i].rid, g)) for i in order for g in range(G))) if G else 1
        words = tokens + token_src + positions + seq_of + q_start + seq_lens + state_slots + want_rows
        offs = {}
        o = 0
        for name, n in (("tokens", N), ("token_src", N), ("positions", N), ("seq_of", N), ("q_start", S + 1),
                        ("seq_lens", S), ("state_slots", S), ("want", R)):
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
            sm += [-1] * n_pad
            bt += [-1] * (n_pad * max_blocks)
            words += sm + bt
            offs[f"slot_map{g}"] = (o, N)
            offs[f"block_table{g}"] = (o + N, S * max_blocks)
            o += N + S * max_blocks
        if extra:
            extra = list(extra) + [0] * (8 * n_pad if pad_to is not None else 0)
            words += extra
            offs["extra"] = (o, len(extra))
        meta = dict(N=N, S=S, R=R, G=G, max_blocks=max_blocks, n_decode=sum(1 for e in entries if len(e.tokens) == 1) + n_pad,
                    q_start=q_start, seq_lens=seq_lens, state_slots=state_slots)
        return words, offs, meta

    def _context(self, dev, offs, meta, arena) -> StepContext:
        def view(name):
            a, n = offs[name]
            return dev[a:a + n]
        N, S, G, max_blocks = meta["N"], meta["S"], meta["G"], meta["max_blocks"]
        ctx = StepContext()
        ctx.device = self.device
        ctx.dtype = self.model.dtype
        ctx.n_tokens, ctx.n_seqs, ctx.n_decode = N, S, meta["n_decode"]
        ctx.tokens, ctx.positions, ctx.seq_of_token = view("tokens"), view("positions"), view("seq_of")
        ctx.token_src = view("token_src")
        ctx.q_start, ctx.seq_lens, ctx.state_slots = view("q_start"), view("seq_lens"), view("state_slots")
        ctx.q_start_host, ctx.seq_lens_host, ctx.state_slots_host = meta["q_start"], meta["seq_lens"], meta["state_slots"]
        ctx.max_query_len = max(meta["q_start"][s + 1] - meta["q_start"][s] for s in range(S))
        ctx.max_seq_len = max(meta["seq_lens"])
        ctx.block_tables = [view(f"block_table{g}").view(S, max_blocks) for g in range(G)]
        ctx.slot_maps = [view(f"slot_map{g}") for g in range(G)]
        ctx.cache = self.cache
        ctx._arena = arena
        ctx.extra = view("extra") if "extra" in offs else None
        ctx.want_rows = view("want")
        return ctx

    # ---- decode-only steps replayed from a HIP graph ----------------------------------------------
    def _run_graph(self, entries, starts, sample_records):
        """A step of one-token sequences only has a fixed shape once it is padded to a bucket
        size, so its kernels (model and sampling) are recorded once per bucket and replayed.
        Only the step's integers change: they are copied into the bucket's own buffer first."""
        from ..kernels import ops
        S = len(entries)
        bucket = 1
        while bucket < S:
            bucket *= 2
        order = list(range(S))
        words, offs, meta = self._pack(entries, order, starts, pad_to=bucket, max_blocks=self.max_blocks_cap,
                                       extra=sample_records)
        st = self._graphs.get(bucket)
        if st is None:
            st = {"dev": torch.empty(len(words), dtype=torch.int32, device=self.device),
                  "host": torch.empty(len(words), dtype=torch.int32, pin_memory=True),
                  "arena": Arena(self.device), "graph": None, "copied": None}
            self._graphs[bucket] = st
        assert st["dev"].numel() == len(words), "a bucket's layout is fixed"
        if st["copied"] is not None:
            st["copied"].synchronize()
        st["host"].copy_(torch.tensor(words, dtype=torch.int32))
        st["dev"].copy_(st["host"], non_blocking=True)
        st["copied"] = torch.cuda.Event()
        st["copied"].record()
        ctx = self._context(st["dev"], offs, meta, st["arena"])
        self.last_ctx = ctx

        sampled = self.sampled[:bucket]

        def body():
            ops.take_tokens(ctx.tokens, ctx.token_src, self.sampled, self.model.config.vocab_size)
            logits = self.model.forward(ctx, ctx.want_rows, bucket)
            ops.sample(logits, ctx.extra, sampled)
            return logits

        if st["graph"] is None:
            st["logits"] = body()                      # eager once: sizes the bucket's scratch buffers
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                st["logits"] = body()
            st["graph"] = g
            # the eager run above already did this step's work; the recorded graph is used from the next step on
        else:
            st["graph"].replay()
        ctx.sampled = sampled[:S]
        return st["logits"][:S], ctx
