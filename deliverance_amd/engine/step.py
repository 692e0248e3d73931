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

import numpy as np
import torch

from ..cache.manager import OutOfPages
from ..models.causal_lm import CausalLM
from ..parts.base import Arena, StepContext
from ..sampling.sampler import RECORD_WORDS
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


class StepPacker:
    """The host side of a step: where each array of the step lies in its one buffer of integers,
    and the values that go there.  It reads the cache manager only, so it runs without a GPU."""

    def __init__(self, manager, n_groups: int, page_size: int):
        self.manager = manager
        self.n_groups = n_groups
        self.page_size = page_size

    def layout(self, entries, order, pad_to, max_blocks, extra):
        """Where each array of the step lies in its one buffer of integers: tokens, where a token
        comes from, positions, sequence ids, row starts, lengths, state slots, wanted rows, then
        per cache group the cache row of every token and the block tables, then ``extra``.  With
        ``pad_to`` the step is filled up with empty one-token sequences (length 0, no cache row),
        so that its shape is fixed."""
        mgr = self.manager
        S_real = len(entries)
        n_pad = 0 if pad_to is None else pad_to - S_real
        N = sum(len(e.tokens) for e in entries) + n_pad
        S = S_real + n_pad
        R = sum(len(e.want) for e in entries) + n_pad
        G = self.n_groups
        if max_blocks is None:
            max_blocks = max(1, max(len(mgr.table(e.rid, g)) for e in entries for g in range(G))) if G else 1
        n_extra = 0 if not extra else len(extra) + RECORD_WORDS * n_pad
        offs = {}
        o = 0
        for name, n in (("tokens", N), ("token_src", N), ("positions", N), ("seq_of", N), ("q_start", S + 1),
                        ("seq_lens", S), ("state_slots", S), ("want", R)):
            offs[name] = (o, n)
            o += n
        for g in range(G):
            offs[f"slot_map{g}"] = (o, N)
            offs[f"block_table{g}"] = (o + N, S * max_blocks)
            o += N + S * max_blocks
        if n_extra:
            offs["extra"] = (o, n_extra)
            o += n_extra
        meta = dict(N=N, S=S, R=R, G=G, max_blocks=max_blocks, n_pad=n_pad,
                    n_decode=sum(1 for e in entries if len(e.tokens) == 1) + n_pad)
        return offs, meta, o

    def fill(self, buf, offs, meta, entries, order, starts, extra):
        """Write the step's integers into ``buf`` (a numpy view of pinned memory).  Long portions
        are written as arrays, single tokens as scalars."""
        mgr = self.manager
        ps = self.page_size

        def view(name):
            a, n = offs[name]
            return buf[a:a + n]
        tok, src, pos, seq = view("tokens"), view("token_src"), view("positions"), view("seq_of")
        q_start_v, seq_lens_v, state_v, want_v = view("q_start"), view("seq_lens"), view("state_slots"), view("want")
        G, mb, n_pad = meta["G"], meta["max_blocks"], meta["n_pad"]
        sms = [view(f"slot_map{g}") for g in range(G)]
        bts = [view(f"block_table{g}") for g in range(G)]
        for bt in bts:
            bt[:] = -1
        q_start, seq_lens, state_slots = [0], [], []
        row0 = {}
        row = 0
        for s, i in enumerate(order):
            e = entries[i]
            n = len(e.tokens)
            st = starts[e.rid]
            row0[i] = row
            if n == 1:
                tok[row] = e.tokens[0]
                src[row] = -1 if e.from_sampled is None else e.from_sampled
                pos[row] = st
                seq[row] = s
            else:
                tok[row:row + n] = e.tokens
                src[row:row + n] = -1
                pos[row:row + n] = np.arange(st, st + n, dtype=np.int32)
                seq[row:row + n] = s
            for g in range(G):
                t = mgr.table(e.rid, g)
                if n == 1:
                    page = t[st // ps]
                    if page < 0:
                        raise StepError(f"position {st} of {e.rid!r} lies in a page that was given back")
                    sms[g][row] = page * ps + st % ps
                else:
                    sms[g][row:row + n] = mgr.slots_for(e.rid, g, st, n)
                bts[g][s * mb:s * mb + len(t)] = t
            row += n
            q_start.append(row)
            seq_lens.append(st + n)
            state_slots.append(mgr.state_slot(e.rid))
        S_real = len(entries)
        r = 0
        for i, e in enumerate(entries):
            for w in e.want:
                want_v[r] = row0[i] + int(w)
                r += 1
        for k in range(n_pad):          # empty one-token sequences
            tok[row] = 0; src[row] = -1; pos[row] = 0; seq[row] = S_real + k
            for g in range(G):
                sms[g][row] = -1
            want_v[r] = row
            r += 1
            row += 1
            q_start.append(row); seq_lens.append(0); state_slots.append(-1)
        q_start_v[:] = q_start
        seq_lens_v[:] = seq_lens
        state_v[:] = state_slots
        if "extra" in offs:
            ex = view("extra")
            ex[:len(extra)] = extra
            ex[len(extra):] = 0
        meta.update(q_start=q_start, seq_lens=seq_lens, state_slots=state_slots)


class StepRunner:
    def __init__(self, model: CausalLM, cache: DeviceCache, use_graphs: bool = False, max_graph_batch: int = 256,
                 kernels: str = "tuned", native_step: bool = True):
        self.model = model
        self.cache = cache
        self.kernels = kernels                       # "tuned" | "reference" (EngineConfig.kernels)
        # the layer loop in one call into the library, where the model's parts allow it (engine/native_step.py)
        self.native = None
        if native_step:
            from .native_step import NativeStep
            if NativeStep.takes(model, cache, kernels):
                self.native = NativeStep(model, cache)
        # hook(layer, stage, tensor) for named intermediates of every step; steps then run kernel by
        # kernel, never from a recorded graph
        self.debug_hook = None
        self.device = model.device
        self.arena = Arena(self.device)
        self.packer = StepPacker(cache.manager, len(cache.groups), cache.page_size)
        self._layout, self._fill = self.packer.layout, self.packer.fill
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
    def _staging_for(self, n: int):
        """The pinned buffer (as a numpy view) that the step's ``n`` integers are written into."""
        if self._staging is None or self._staging.numel() < n:
            cap = max(4096, 2 * n)
            self._staging = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._staging_np = self._staging.numpy()
            self._staging_dev = torch.empty(cap, dtype=torch.int32, device=self.device)
            self._copied = None
        if self._copied is not None:
            self._copied.synchronize()       # the last step's copy has read the pinned buffer
        return self._staging_np[:n]

    def _upload(self, n: int) -> torch.Tensor:
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
            if len(e.tokens) <= 8:
                bad = [t for t in e.tokens if not (0 <= int(t) < cfg.vocab_size)]
            else:
                arr = np.asarray(e.tokens, dtype=np.int64)
                bad = arr[(arr < 0) | (arr >= cfg.vocab_size)].tolist()
            if bad:
                raise StepError(f"request {e.rid!r}: token id {bad[0]} is outside the vocabulary of {cfg.vocab_size}")
            for w in e.want:
                if not (0 <= int(w) < len(e.tokens)):
                    raise StepError(f"request {e.rid!r}: wanted place {w} is outside its {len(e.tokens)} tokens")
            if e.from_sampled is not None and not (len(e.tokens) == 1 and 0 <= e.from_sampled < self.sampled.numel()):
                raise StepError(f"request {e.rid!r}: only a single token can come from the sampled tokens")

        starts = {}
        opened = []
        if reserved:
            for e in entries:               # the entry's tokens are the last positions that were reserved
                starts[e.rid] = mgr.length(e.rid) + mgr.pending(e.rid) - len(e.tokens)
                if starts[e.rid] < mgr.length(e.rid):
                    raise StepError(f"request {e.rid!r} brings {len(e.tokens)} tokens, {mgr.pending(e.rid)} are reserved")
        else:
            done = []
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
        from ..profiler import KernelProfiler
        graph_ok = (sample_records is not None and n_decode == len(entries) and self.use_graphs
                    and self.debug_hook is None and not KernelProfiler.enabled
                    and len(entries) <= self.max_graph_batch and all(list(e.want) == [0] for e in entries))
        from ..kernels import ops
        try:
            with ops.kernel_mode_scope(self.kernels):
                if graph_ok:
                    logits, ctx = self._run_graph(entries, starts, sample_records)
                else:
                    logits, ctx = self._run_eager(entries, order, starts, sample_records)
        except Exception:
            # A launch that was refused (a size no kernel takes) leaves nothing half-done on the host:
            # what this call reserved goes back, requests it opened are closed.  A caller that
            # reserved itself decides what becomes of its requests.
            if not reserved:
                for e in entries:
                    mgr.rollback(e.rid)
                for rid in opened:
                    mgr.close(rid)
            raise
        if not reserved:                 # who reserves commits: the scheduler does it for its batches
            for e in entries:
                mgr.commit(e.rid)
        return logits, ctx

    def _run_eager(self, entries, order, starts, sample_records):
        from ..kernels import ops
        offs, meta, n_words = self._layout(entries, order, pad_to=None, max_blocks=None, extra=sample_records)
        self._fill(self._staging_for(n_words), offs, meta, entries, order, starts, sample_records)
        dev = self._upload(n_words)
        ctx = self._context(dev, offs, meta, self.arena)
        ctx.debug_hook = self.debug_hook
        self.last_ctx = ctx
        R = meta["R"]
        if any(e.from_sampled is not None for e in entries):
            ops.take_tokens(ctx.tokens, ctx.token_src, self.sampled, self.model.config.vocab_size)
        logits = self._forward(ctx, ctx.want_rows if R else None, R)
        return logits, ctx

    def _forward(self, ctx, want_rows, n_want):
        """The model's forward pass of this step: from C++ in one call, or part by part (always with the
        debug hook or the kernel profiler, which look between the kernels)."""
        from ..profiler import KernelProfiler
        if self.native is not None and ctx.debug_hook is None and not KernelProfiler.enabled:
            return self.native.forward(ctx, want_rows, n_want)
        return self.model.forward(ctx, want_rows, n_want)

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
        offs, meta, n_words = self._layout(entries, order, pad_to=bucket, max_blocks=self.max_blocks_cap,
                                           extra=sample_records)
        st = self._graphs.get(bucket)
        if st is None:
            host = torch.empty(n_words, dtype=torch.int32, pin_memory=True)
            st = {"dev": torch.empty(n_words, dtype=torch.int32, device=self.device),
                  "host": host, "host_np": host.numpy(),
                  "arena": Arena(self.device), "graph": None, "copied": None}
            self._graphs[bucket] = st
        assert st["dev"].numel() == n_words, "a bucket's layout is fixed"
        if st["copied"] is not None:
            st["copied"].synchronize()
        self._fill(st["host_np"], offs, meta, entries, order, starts, sample_records)
        st["dev"].copy_(st["host"], non_blocking=True)
        st["copied"] = torch.cuda.Event()
        st["copied"].record()
        ctx = self._context(st["dev"], offs, meta, st["arena"])
        self.last_ctx = ctx

        sampled = self.sampled[:bucket]

        def body():
            ops.take_tokens(ctx.tokens, ctx.token_src, self.sampled, self.model.config.vocab_size)
            logits = self._forward(ctx, ctx.want_rows, bucket)
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
