"""The engine as a user sees it: load a model folder, generate tokens for prompts.

In the reference's manner (README.md:84-107; core/src/test/java/io/teknek/deliverance/
integration/Gpt2IT.java:25-36)::

    model = AutoModelForCausalLM.from_pretrained(folder, dtype="bfloat16")
    response = model.generate(prompt_ids, GeneratorParameters().with_temperature(0.0)
                              .with_ntokens(500).with_max_tokens(150), on_token)

``Response`` carries what the reference's does for an engine that works on token ids
(core/.../generator/Response.java:10-22): generated tokens, finish reason, prompt tokens and
the three timings.  Several prompts may be given at once; they are batched continuously.
"""
from __future__ import annotations

import struct
import time
from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence, Union

import torch

from ..config.engine_config import EngineConfig
from ..kernels import ops
from ..models.causal_lm import CausalLM, load_model
from ..profiler import InferenceProfiler
from ..sampling.params import GeneratorParameters
from ..sampling.sampler import RECORD_WORDS, device_record
from .device_cache import DeviceCache
from .scheduler import RUNNING, Request, Scheduled, Scheduler
from .step import StepEntry, StepRunner

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


@dataclass
class Response:
    generated_tokens: List[int]
    finish_reason: str                  # "length" | "stop" | "error" | "cancelled"
    prompt_tokens: int
    time_to_first_token_ms: float = 0.0
    avg_time_per_token_ms: float = 0.0
    total_time_ms: float = 0.0
    top_logprobs: List[list] = field(default_factory=list)
    error: Optional[str] = None
    preemptions: int = 0


class _InFlight:
    """A step that has been launched: its batch, and where its sampled tokens arrive."""

    def __init__(self, batch: List[Scheduled], samplers: List[Scheduled]):
        self.batch = batch
        self.samplers = samplers
        self.tokens_host: Optional[torch.Tensor] = None      # pinned; valid once ``ready`` has passed
        self.ready: Optional[torch.cuda.Event] = None
        self.lp = None                                       # (indices, values) of the top log-probabilities


class CausalLanguageModel:
    """A loaded model with its cache, step function and scheduler on one GPU."""

    def __init__(self, model: CausalLM, engine_config: EngineConfig):
        if not torch.cuda.is_available():
            raise RuntimeError("deliverance_amd runs on a GPU only; no device is visible")
        self.model = model
        self.config = model.config
        self.engine_config = engine_config
        needs = model.cache_needs()
        tokens = engine_config.max_cached_tokens
        n_slots = engine_config.state_slots if engine_config.state_slots is not None else engine_config.max_num_seqs
        if tokens is None:
            free, _ = torch.cuda.mem_get_info(model.device)
            tokens = DeviceCache.tokens_for_budget(needs, model.dtype, int(free * 0.5), n_slots)
            tokens = min(tokens, engine_config.max_num_seqs * model.config.max_positions)
            tokens = max(tokens, engine_config.page_size)
        self.cache = DeviceCache(needs, model.dtype, model.device, engine_config.page_size, tokens, n_slots,
                                 poison_freed=engine_config.poison_freed_pages)
        self.runner = StepRunner(model, self.cache, use_graphs=engine_config.use_graphs,
                                 max_graph_batch=max(engine_config.max_num_seqs, 1), kernels=engine_config.kernels,
                                 native_step=engine_config.native_step)
        self.scheduler = Scheduler(self.cache.manager, model.config.max_positions, model.config.eos_token_ids,
                                   engine_config.max_num_seqs, engine_config.max_batch_tokens,
                                   engine_config.max_chunk, on_open=self.cache.reset_state)
        self._next_id = 0
        self._callbacks: Dict[Hashable, Callable] = {}
        self._inflight: Optional[_InFlight] = None
        self._ended_outside: List[Request] = []       # cancelled between steps; the next step() reports them
        # hook(batch, logits): every launched step's scheduled portions and its logits on the device
        # (row i: the i-th portion that samples), before anything is read back; for tests and diagnosis
        self.logits_hook: Optional[Callable] = None
        self._n_launched = 0
        n = 2 * max(engine_config.max_num_seqs, 64)
        self._token_bufs = [torch.empty(n, dtype=torch.int32, pin_memory=True) for _ in range(3)]

    # ---- lower level: requests and steps -------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[GeneratorParameters] = None,
                    rid: Optional[Hashable] = None, on_token: Optional[Callable] = None) -> Hashable:
        if rid is None:
            rid = self._next_id
            self._next_id += 1
        for t in prompt:
            if not (0 <= int(t) < self.config.vocab_size):
                raise ValueError(f"token id {t} is outside the vocabulary of {self.config.vocab_size}")
        self.scheduler.add(rid, [int(t) for t in prompt], params or GeneratorParameters())
        if on_token is not None:
            self._callbacks[rid] = on_token
        return rid

    def has_work(self) -> bool:
        return self.scheduler.has_work() or self._inflight is not None or bool(self._ended_outside)

    def cancel(self, rid: Hashable) -> bool:
        """End a request now, between two steps (also from inside an ``on_token`` callback); True when
        it was waiting or running.  Its pages and state slot go back at once, also those that a step
        which is still running holds for it: that step's work for the request is dropped when the
        step is read, and whoever gets the pages next writes them after that step in stream order.
        The request ends with ``finish_reason = "cancelled"`` and is reported by the next ``step()``.
        The reference stops a generation between two tokens likewise
        (core/src/main/java/io/teknek/deliverance/model/GenerationEngine.java:221-225)."""
        before = len(self.scheduler.finished)
        if not self.scheduler.cancel(rid):
            return False
        self._ended_outside += self.scheduler.finished[before:]
        self._callbacks.pop(rid, None)
        return True

    def set_layer_debug_hook(self, hook: Optional[Callable]) -> None:
        """``hook(layer, stage, tensor)`` receives copies of named intermediates of every step (layer -1,
        "input": the embedding; per layer "query_projection", "key_projection", "value_projection",
        "attention_value", "attention_output", "post_attention_residual", "post_ff_residual", "layer_output"), as the
        reference's ``setLayerDebugHook`` does (core/.../model/AbstractModel.java:122-128,505-515,1100-1107).
        While a hook is set, steps run kernel by kernel (no recorded graphs) and slowly."""
        self.runner.debug_hook = hook

    def step(self) -> List[Request]:
        """One scheduler decision and one model step with its sampling.  Returns the requests
        whose end became known in this call.

        A step may be left running when the call returns.  The next call then first launches the
        step after it (``Scheduler.schedule_ahead``; tokens that are still being sampled are taken
        on the device) and only then reads the older step's tokens, so the host's work for one
        step runs beside the device's work for the step before.  When the next step cannot be
        decided ahead (pages are short), the older step is read first, as without this."""
        done: List[Request] = self._ended_outside
        self._ended_outside = []
        if self._inflight is not None:
            ahead = self._launch_ahead(self._inflight)
            done += self._retire(self._inflight)
            self._inflight = ahead
            if ahead is not None:
                return done
        before = len(self.scheduler.finished)
        with InferenceProfiler.timer("scheduler.schedule"):
            batch: List[Scheduled] = self.scheduler.schedule()
        done += self.scheduler.finished[before:]         # requests that failed in scheduling
        if not batch:
            return done
        flight = self._launch(batch, None)
        if self._may_stay_in_flight(flight):
            self._inflight = flight
        else:
            done += self._retire(flight)
        return done

    def drain(self) -> List[Request]:
        """Read the step that is still running, if there is one."""
        if self._inflight is None:
            return []
        flight, self._inflight = self._inflight, None
        return self._retire(flight)

    def _may_stay_in_flight(self, flight: "_InFlight") -> bool:
        return self.engine_config.run_ahead and flight.lp is None

    def _launch_ahead(self, prev: "_InFlight") -> Optional["_InFlight"]:
        if any(s.request.params.log_probs and s.request.params.top_log_probs > 0 for s in prev.batch):
            return None
        with InferenceProfiler.timer("scheduler.schedule"):
            batch = self.scheduler.schedule_ahead(prev.batch)
        if batch is None:
            return None
        row = {id(s.request): i for i, s in enumerate(prev.samplers)}
        return self._launch(batch, row)

    def _launch(self, batch: List[Scheduled], sampled_row: Optional[Dict[int, int]]) -> "_InFlight":
        """Put one step on the device: model, sampling, and the copy of the sampled tokens to the
        host.  An entry whose token the host does not know yet takes the one the step before
        sampled for the same request (row ``sampled_row[id(request)]`` of the runner's sampled
        tokens)."""
        V = self.config.vocab_size
        entries = []
        records: List[int] = []
        samplers: List[Scheduled] = []
        for s in batch:
            req = s.request
            if s.start + s.n <= req.n_tokens:
                entries.append(StepEntry(req.rid, req.tokens_from(s.start, s.n), [s.n - 1] if s.samples else []))
            else:       # the one token that the running step is still sampling
                assert sampled_row is not None and s.n == 1 and s.start == req.n_tokens
                entries.append(StepEntry(req.rid, [0], [0], from_sampled=sampled_row[id(req)]))
            if s.samples:
                records += struct.unpack(f"<{RECORD_WORDS}i", device_record(req.params, req.rng, V))
                samplers.append(s)
        decode_only = all(s.n == 1 for s in batch)
        try:
            with InferenceProfiler.timer("generation.decode" if decode_only else "generation.prefill"):
                logits, ctx = self.runner.run(entries, reserved=True, sample_records=records or None)
        except Exception as e:
            # a step that could not be put on the device: its requests end with an error and give
            # back what the scheduler had reserved for them
            for s in batch:
                self.scheduler._fail(s.request, f"the step could not be launched: {e}")
            raise
        if self.logits_hook is not None:
            self.logits_hook(batch, logits)
        InferenceProfiler.counter("engine.batch_tokens", sum(s.n for s in batch))
        flight = _InFlight(batch, samplers)
        if not samplers:
            return flight
        R = len(samplers)
        out = getattr(ctx, "sampled", None)           # a replayed graph has sampled already
        if out is None:
            out = self.runner.sampled[:R]
            ops.sample(logits, ctx.extra, out)
        want_lp = [s for s in samplers if s.request.params.log_probs and s.request.params.top_log_probs > 0]
        if want_lp:
            n = max(s.request.params.top_log_probs for s in want_lp)
            idx = torch.empty((R, n), dtype=torch.int32, device=self.model.device)
            val = torch.empty((R, n), dtype=torch.float32, device=self.model.device)
            ops.top_logprobs(logits, ctx.extra, n, idx, val)
            flight.lp = (idx, val)
        host = self._token_bufs[self._n_launched % len(self._token_bufs)]
        self._n_launched += 1
        if host.numel() < R:
            host = torch.empty(2 * R, dtype=torch.int32, pin_memory=True)
            self._token_bufs[(self._n_launched - 1) % len(self._token_bufs)] = host
        host[:R].copy_(out, non_blocking=True)
        flight.tokens_host = host
        flight.ready = torch.cuda.Event()
        flight.ready.record()
        return flight

    def _retire(self, flight: "_InFlight") -> List[Request]:
        """Wait for a launched step's tokens, book it with the scheduler, tell the callbacks."""
        sampled: Dict[Hashable, int] = {}
        samplers = flight.samplers
        if samplers:
            with InferenceProfiler.timer("sampler.sample"):
                flight.ready.synchronize()                   # the step's one synchronisation
                host = flight.tokens_host[:len(samplers)].tolist()
            lp = None if flight.lp is None else (flight.lp[0].cpu(), flight.lp[1].cpu())
            for i, s in enumerate(samplers):
                if s.request.state != RUNNING:
                    continue                                 # ended while this step was running
                sampled[s.request.rid] = host[i]
                p = s.request.params
                if lp is not None and p.log_probs and p.top_log_probs > 0:
                    k = p.top_log_probs
                    s.request.top_logprobs.append(list(zip(lp[0][i, :k].tolist(), lp[1][i, :k].tolist())))
        live = [s for s in samplers if s.request.state == RUNNING]
        done = self.scheduler.complete(flight.batch, sampled)
        now = time.perf_counter()
        for s in live:
            cb = self._callbacks.get(s.request.rid)
            if cb is not None:
                cb(sampled[s.request.rid], s.request.rid, (now - s.request.t_arrival) * 1e3)
        for r in done:
            self._callbacks.pop(r.rid, None)
        return done

    # ---- the entry point ---------------------------------------------------------------------
    def generate(self, prompts: Union[Sequence[int], Sequence[Sequence[int]]],
                 params: Union[None, GeneratorParameters, Sequence[GeneratorParameters]] = None,
                 on_token: Optional[Callable] = None) -> Union[Response, List[Response]]:
        """Generate for one prompt (a list of token ids) or several (a list of lists).
        ``on_token(token, request_index, ms_since_arrival)`` is called for every new token, as
        the reference's ``GenerateEvent.emit`` is (core/.../model/GenerateEvent.java:3-12)."""
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        plist = [prompts] if single else list(prompts)
        if params is None or isinstance(params, GeneratorParameters):
            pl = [params or GeneratorParameters()] * len(plist)
        else:
            pl = list(params)
            if len(pl) != len(plist):
                raise ValueError("one GeneratorParameters per prompt is needed")
        rids = []
        for i, (pr, pa) in enumerate(zip(plist, pl)):
            cb = None if on_token is None else (lambda tok, rid, ms, i=i: on_token(tok, i, ms))
            rids.append(self.add_request(pr, pa, on_token=cb))
        mine = set(rids)
        got: Dict[Hashable, Request] = {}
        while len(got) < len(rids):
            if not self.has_work():
                raise RuntimeError("the scheduler ran out of work before every request finished")
            for r in self.step():
                if r.rid in mine:
                    got[r.rid] = r
        self.drain()                 # a step launched ahead for requests that have ended since
        out = [self._response(got[r]) for r in rids]
        for r in rids:
            self.scheduler.finished.remove(got[r])
        return out[0] if single else out

    @staticmethod
    def _response(r: Request) -> Response:
        """Timing as the reference computes it (core/.../model/GenerationEngine.java:249-268)."""
        end = r.t_finish or time.perf_counter()
        total = (end - r.t_arrival) * 1e3
        ttft = ((r.t_first_token or end) - r.t_arrival) * 1e3
        n = len(r.output)
        return Response(list(r.output), r.finish_reason or "error", len(r.prompt), ttft,
                        total / n if n else 0.0, total, list(r.top_logprobs), r.error, r.n_preempted)

    def stats(self) -> dict:
        d = dict(self.scheduler.counters)
        d.update(self.cache.manager.stats())
        return d


class AutoModelForCausalLM:
    """``from_pretrained`` reads config.json, picks the model by its architecture name and loads
    the tensors by name (the reference: core/.../model/AutoModelForCausaLm.java:92-103,457-520)."""

    @staticmethod
    def from_pretrained(folder: str, dtype: str = "bfloat16", engine_config: Optional[EngineConfig] = None,
                        **kwargs) -> CausalLanguageModel:
        import deliverance_amd.models  # noqa: F401  (registers the architectures)
        ec = engine_config or EngineConfig(dtype=dtype, **kwargs)
        model = load_model(folder, _TORCH_DTYPE[ec.dtype], ec.device)
        return CausalLanguageModel(model, ec)
