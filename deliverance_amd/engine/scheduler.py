"""The scheduler: admits requests, cuts prompts into portions under a token budget, keeps the
running requests decoding, finishes and frees.  Pure host code: it sees token counts, the
cache manager's bookkeeping and sampled tokens, never a tensor.

The reference runs one request at a time on the caller's thread: the prompt in chunks of 512
(core/src/main/java/io/teknek/deliverance/model/AbstractModel.java:87,1022-1031), then one
token per forward (core/.../model/GenerationEngine.java:138-159), with the stop rules of
GenerationEngine.java:189-219 and the request limits of :98-104.  Those rules are kept per
request; batching across requests, the token budget and the behaviour when pages run out are
this engine's own:

* Every step first gives one token to each running request that is decoding, then portions of
  prompts to running requests still prefilling (oldest first), then admits waiting requests.
* A portion is at most ``max_chunk`` tokens, at most what is left of the budget, and at most
  what the free pages can hold.
* When a running request cannot get a page, the most recently admitted running request is
  preempted: its pages go back and it returns to the head of the waiting queue to be computed
  again from its tokens (prompt and what it has generated).  A request that is alone and still
  cannot fit fails with ``finish_reason = "error"``.
* ``schedule_ahead`` decides the step after one that is still running, before its tokens are
  known: requests that sampled there decode the token that is still on the device (those that end
  by length leave), prompts get their next portions, waiting requests are admitted.  Only when
  pages run short does it decline: preemption is decided with the tokens known.  A request that
  turns out to have sampled an end token has then one step too many in flight; its result is
  dropped when that step is booked.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Dict, Hashable, List, Optional

from ..cache.manager import CacheManager
from ..sampling.params import GeneratorParameters
from ..sampling.sampler import JavaRandom

WAITING, RUNNING, FINISHED = "waiting", "running", "finished"
FINISH_LENGTH, FINISH_STOP, FINISH_ERROR, FINISH_CANCELLED = "length", "stop", "error", "cancelled"


@dataclass(eq=False)
class Request:
    rid: Hashable
    prompt: List[int]
    params: GeneratorParameters
    limit: int                                    # positions the request may reach (ntokens)
    output: List[int] = field(default_factory=list)
    n_computed: int = 0                           # tokens whose keys and values are cached
    state: str = WAITING
    finish_reason: Optional[str] = None
    error: Optional[str] = None
    rng: JavaRandom = None
    n_preempted: int = 0
    t_arrival: float = 0.0
    t_first_token: Optional[float] = None
    t_finish: Optional[float] = None
    top_logprobs: List[list] = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        return len(self.prompt) + len(self.output)

    def token_at(self, i: int) -> int:
        return self.prompt[i] if i < len(self.prompt) else self.output[i - len(self.prompt)]

    def tokens_from(self, start: int, n: int) -> List[int]:
        return [self.token_at(i) for i in range(start, start + n)]


@dataclass
class Scheduled:
    request: Request
    start: int            # first position of the portion
    n: int                # tokens in the portion
    samples: bool         # the portion ends at the request's last token, so a token is sampled


class SchedulerError(ValueError):
    pass


class Scheduler:
    def __init__(self, cache: CacheManager, max_positions: int, eos_token_ids=(), max_num_seqs: int = 64,
                 max_batch_tokens: int = 2048, max_chunk: int = 512,
                 on_open: Optional[Callable[[int], None]] = None):
        self.cache = cache
        self.max_positions = max_positions
        self.eos = set(eos_token_ids)
        self.max_num_seqs = max_num_seqs
        self.max_batch_tokens = max_batch_tokens
        self.max_chunk = max_chunk
        self.on_open = on_open                       # told the state slot of a request that starts
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self.counters = {"steps": 0, "batch_tokens": 0, "preemptions": 0, "admitted": 0, "finished": 0}

    # ---- admission ---------------------------------------------------------------------------
    def add(self, rid: Hashable, prompt: List[int], params: GeneratorParameters) -> Request:
        """The reference's preconditions (GenerationEngine.java:98-104): the prompt is shorter
        than the context and than ``ntokens``, and ``ntokens`` does not exceed the context."""
        params.validate()
        if not prompt:
            raise SchedulerError("a prompt needs at least one token")
        ntokens = params.ntokens if params.ntokens is not None else self.max_positions
        if ntokens > self.max_positions:
            raise SchedulerError(f"ntokens {ntokens} exceed config length {self.max_positions}")
        if not (len(prompt) < self.max_positions and len(prompt) < ntokens):
            raise SchedulerError(f"Prompt exceeds ntokens ({len(prompt)} tokens, ntokens {ntokens})")
        if any(r.rid == rid for r in list(self.waiting) + self.running):
            raise SchedulerError(f"request {rid!r} is already queued")
        req = Request(rid, list(prompt), params, ntokens, rng=JavaRandom(params.seed), t_arrival=time.perf_counter())
        self.waiting.append(req)
        return req

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- one step's batch ----------------------------------------------------------------------
    def _fit(self, req: Request, n: int, opened: bool) -> int:
        """The largest portion <= n whose pages are free right now."""
        ps = self.cache.page_size
        if opened:
            # every group has a table of the same length; the smallest is what counts should they differ
            have = min((len(self.cache.table(req.rid, g)) for g in range(len(self.cache.groups))), default=None)
            have = 10 ** 9 if have is None else have * ps
            base = self.cache.length(req.rid) + self.cache.pending(req.rid)
        else:
            have, base = 0, 0
        free = min((p.n_free for p in self.cache.pools), default=10 ** 9)
        room = max(0, have - base) + free * ps
        return min(n, room)

    def _preempt(self, victim: Request) -> None:
        self.cache.close(victim.rid)
        self.running.remove(victim)
        victim.state = WAITING
        victim.n_computed = 0
        victim.n_preempted += 1
        self.waiting.appendleft(victim)
        self.counters["preemptions"] += 1

    def _fail(self, req: Request, why: str) -> None:
        if req.rid in self.cache:
            self.cache.close(req.rid)
        if req in self.running:
            self.running.remove(req)
        req.state, req.finish_reason, req.error = FINISHED, FINISH_ERROR, why
        req.t_finish = time.perf_counter()
        self.finished.append(req)
        self.counters["finished"] += 1

    def _admit(self, batch: List[Scheduled], budget: int) -> None:
        """Admission, in arrival order, never at a running request's cost."""
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs and self.cache.can_open():
            req = self.waiting[0]
            want = min(req.n_tokens, budget, self.max_chunk)
            n = self._fit(req, want, False)
            if n == 0:
                if not self.running and not batch:
                    self.waiting.popleft()
                    self._fail(req, "the cache pool cannot hold a single page for the request")
                    continue
                break
            self.waiting.popleft()
            slot = self.cache.open(req.rid)
            if self.on_open is not None:
                self.on_open(slot)
            req.state = RUNNING
            self.running.append(req)
            self.counters["admitted"] += 1
            start = self.cache.extend(req.rid, n)
            batch.append(Scheduled(req, start, n, start + n == req.n_tokens))
            budget -= n

    def schedule(self) -> List[Scheduled]:
        """Pick this step's work and reserve its cache positions."""
        budget = self.max_batch_tokens
        batch: List[Scheduled] = []
        # running requests: the ones that decode first, then the ones still in their prompt
        for phase in (1, 0):
            for req in list(self.running):
                if req not in self.running:
                    continue                        # preempted a moment ago
                left = req.n_tokens - req.n_computed
                if (left == 1) != bool(phase) or budget <= 0:
                    continue
                want = min(left, budget, self.max_chunk)
                n = self._fit(req, want, True)
                while n == 0:
                    victim = self.running[-1]
                    if victim is req:
                        others = any(s.request is not req for s in batch) or len(self.running) > 1
                        if others:
                            self._preempt(req)
                        else:
                            self._fail(req, f"the request needs more cache than the whole pool holds "
                                            f"({req.n_tokens} tokens)")
                        break
                    if any(s.request is victim for s in batch):
                        # the newest request already has its place in this step; the asker waits
                        break
                    self._preempt(victim)
                    n = self._fit(req, want, True)
                if n == 0 or req not in self.running:
                    continue
                start = self.cache.extend(req.rid, n)
                batch.append(Scheduled(req, start, n, start + n == req.n_tokens))
                budget -= n
        self._admit(batch, budget)
        if batch:
            self.counters["steps"] += 1
            self.counters["batch_tokens"] += sum(s.n for s in batch)
        return batch

    # ---- the step after a running one ----------------------------------------------------------
    def _ends_by_length(self, req: Request, more: int) -> bool:
        """Whether the request is done by its length once ``more`` further tokens are appended."""
        p = req.params
        return ((p.max_tokens is not None and len(req.output) + more >= p.max_tokens)
                or req.n_tokens + more > req.limit)

    def schedule_ahead(self, inflight: List[Scheduled]) -> Optional[List[Scheduled]]:
        """The batch that follows ``inflight`` (scheduled, launched, not yet completed), decided
        without its tokens: a request that sampled in ``inflight`` decodes the token that is still on
        the device (unless it ends by length), a request in its prompt gets its next portion, waiting
        requests are admitted as in ``schedule``.  Returns None, with nothing reserved, when a running
        request cannot get all the pages it asks for: who gives way then is decided with the tokens
        known."""
        last = {id(s.request): s for s in inflight}
        G = len(self.cache.pools)
        need = [0] * G
        free = [p.n_free for p in self.cache.pools]
        budget = self.max_batch_tokens
        plan = []
        for phase in (1, 0):
            for req in self.running:
                s = last.get(id(req))
                if s is None:
                    done, total = req.n_computed, req.n_tokens
                else:
                    if s.samples and self._ends_by_length(req, 1):
                        continue                    # ends when ``inflight`` is completed
                    done, total = s.start + s.n, req.n_tokens + (1 if s.samples else 0)
                left = total - done
                if left <= 0:
                    return None
                if (left == 1) != bool(phase) or budget <= 0:
                    continue
                want = min(left, budget, self.max_chunk)
                pages = self.cache.pages_needed(req.rid, want)
                if any(need[g] + pages[g] > free[g] for g in range(G)):
                    return None
                for g in range(G):
                    need[g] += pages[g]
                plan.append((req, done, want, done + want == total))
                budget -= want
        batch = []
        for req, start, n, samples in plan:
            got = self.cache.extend(req.rid, n)
            assert got == start, "reserved positions follow the running step's"
            batch.append(Scheduled(req, start, n, samples))
        self._admit(batch, budget)
        if not batch:
            return None
        self.counters["steps"] += 1
        self.counters["batch_tokens"] += sum(s.n for s in batch)
        return batch

    # ---- after the step ----------------------------------------------------------------------
    def finish_check(self, req: Request, token: int) -> Optional[str]:
        """Stop rules after a token was appended (GenerationEngine.java:189-219,163-173):
        the cap on generated tokens, then an end token, then the position limit."""
        p = req.params
        if p.max_tokens is not None and len(req.output) >= p.max_tokens:
            return FINISH_LENGTH
        if token in self.eos and not p.ignore_eos:
            return FINISH_STOP
        if req.n_tokens > req.limit:
            # The reference's loop decodes positions up to ntokens - 1 and samples after each
            # (GenerationEngine.java:138-159), so the last sampled token would sit at position
            # ntokens and is never computed.
            return FINISH_LENGTH
        return None

    def complete(self, batch: List[Scheduled], sampled: Dict[Hashable, int]) -> List[Request]:
        """Book the step: positions are now cached; sampled tokens are appended; requests that
        are done give their pages back.  Returns the requests that finished."""
        done = []
        now = time.perf_counter()
        for s in batch:
            req = s.request
            if req.state != RUNNING:
                continue
            self.cache.commit(req.rid, s.n)           # a step scheduled ahead may hold a reservation of its own
            req.n_computed = s.start + s.n
            if not s.samples:
                continue
            token = int(sampled[req.rid])
            req.output.append(token)
            if req.t_first_token is None:
                req.t_first_token = now
            reason = self.finish_check(req, token)
            if reason is not None:
                self.cache.close(req.rid)
                self.running.remove(req)
                req.state, req.finish_reason, req.t_finish = FINISHED, reason, now
                self.finished.append(req)
                self.counters["finished"] += 1
                done.append(req)
        return done

    def cancel(self, rid: Hashable) -> bool:
        """Remove a request at a step boundary; what it holds goes back."""
        for req in list(self.waiting):
            if req.rid == rid:
                self.waiting.remove(req)
                req.state, req.finish_reason, req.t_finish = FINISHED, FINISH_CANCELLED, time.perf_counter()
                self.finished.append(req)
                return True
        for req in self.running:
            if req.rid == rid:
                self.cache.close(rid)
                self.running.remove(req)
                req.state, req.finish_reason, req.t_finish = FINISHED, FINISH_CANCELLED, time.perf_counter()
                self.finished.append(req)
                return True
        return False
