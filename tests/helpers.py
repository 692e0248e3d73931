"""Shared pieces of the tests: the two tiny configurations, prompts, trace builders for the
ways of cutting a request into steps, and the comparison with the plain implementation."""
from __future__ import annotations

import functools
import os

import numpy as np

import plain_gpt2

# Two tiny GPT-2 configurations that differ in every size and option.
CONFIG_A = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=2, n_embd=64, n_head=4,
                vocab_size=512, n_positions=128, layer_norm_epsilon=1e-5, activation_function="gelu_new",
                scale_attn_by_inverse_layer_idx=False, bos_token_id=511, eos_token_id=511)
CONFIG_B = dict(architectures=["GPT2LMHeadModel"], model_type="gpt2", n_layer=3, n_embd=96, n_head=2,
                n_inner=200, vocab_size=1000, n_positions=96, layer_norm_epsilon=1e-6,
                activation_function="gelu", scale_attn_by_inverse_layer_idx=True, bos_token_id=0,
                eos_token_id=999)

# Where the GPU tests put their tensors: the GPU, or (DELIVERANCE_SIMT=1) the CPU, where the kernels
# run simulated under guard pages (tests/simt).
SIMT = os.environ.get("DELIVERANCE_SIMT") == "1"
DEVICE = "cpu" if SIMT else "cuda:0"


def trace_session(folder, dtype, max_tokens, page_size=16, poison_freed=False, **options):
    """The engine's trace session on the GPU, or its stand-in on the simulated kernels (which has no
    recorded graphs: ``use_graphs`` is dropped there)."""
    if SIMT:
        from simt import harness
        options.pop("use_graphs", None)
        return harness.SimTraceSession(None, str(folder), dtype, max_tokens, page_size, poison_freed=poison_freed,
                                       **options)
    from deliverance_amd.trace import TraceSession
    return TraceSession(str(folder), dtype, max_tokens, page_size, poison_freed=poison_freed, **options)


def quick(*values, mark="simt_quick"):
    """A parameter of the default selection for the simulated kernels (tests/test_simt.py)."""
    import pytest
    return pytest.param(*values, marks=getattr(pytest.mark, mark))


def skip_in_simulation_if(cond, why="too much arithmetic for the simulated kernels"):
    if SIMT and cond:
        import pytest
        pytest.skip(why)


# Absolute tolerance on 32-bit logits (their magnitude is about 1 on these models).
ATOL = {"float32": 5e-6}


class TinyModel:
    def __init__(self, folder, cfg, seed):
        self.folder = str(folder)
        self.cfg = cfg
        self.seed = seed
        self.plain_cfg, self.W = plain_gpt2.read_model_folder(self.folder)

    @functools.lru_cache(maxsize=None)
    def _logits(self, ids):
        return plain_gpt2.forward_logits(self.plain_cfg, self.W, list(ids))

    def plain_logits(self, ids):
        """[T, V] float64 logits of the whole sequence from the plain implementation."""
        return self._logits(tuple(int(i) for i in ids))

    def prompt(self, length, salt=0):
        rng = np.random.default_rng(1000 * self.seed + 7 * length + salt)
        return [int(t) for t in rng.integers(0, self.cfg["vocab_size"], size=length)]


def make_model(folder, cfg, seed, store_dtype="bfloat16"):
    """A model folder with random weights, stored in bfloat16 or (as openai-community/gpt2 ships) in
    32-bit: those weights are not bfloat16 numbers, so the 32-bit path meets them unrounded and the
    bfloat16 path takes its kernels for 32-bit parameter vectors and tables."""
    import torch
    from deliverance_amd.random_model import random_model
    random_model(str(folder), cfg, seed, {"bfloat16": torch.bfloat16, "float32": torch.float32}[store_dtype])
    return TinyModel(folder, cfg, seed)


# ------------------------------------------------------------------------ trace builders
def trace_whole(rid, ids):
    return [{"step": 0, "entries": [{"id": rid, "tokens": list(ids), "want": list(range(len(ids)))}], "end": [rid]}]


def trace_bulk_then_single(rid, ids, tail=32):
    """All but the last ``tail`` tokens in one step, then one token a step."""
    tail = min(tail, len(ids) - 1)
    head = len(ids) - tail
    steps = [{"step": 0, "entries": [{"id": rid, "tokens": list(ids[:head]), "want": list(range(head))}], "end": []}]
    for i in range(head, len(ids)):
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [ids[i]], "want": [0]}], "end": []})
    steps[-1]["end"] = [rid]
    return steps


def trace_portions(rid, ids, sizes=(7, 2, 13, 3, 5, 2)):
    """Portions of changing size, down to two tokens."""
    steps, pos, k = [], 0, 0
    while pos < len(ids):
        n = min(sizes[k % len(sizes)], len(ids) - pos)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": list(ids[pos:pos + n]),
                                                       "want": list(range(n))}], "end": []})
        pos += n
        k += 1
    steps[-1]["end"] = [rid]
    return steps


def trace_mixed(requests, seed=0, max_live=4, prefill_sizes=(9, 2, 17, 4, 6), decode_tail=12):
    """Up to ``max_live`` requests at a time: portions of some beside single tokens of others;
    requests end and new ones start mid-trace.  ``requests`` is a list of (rid, ids).  The last
    ``decode_tail`` tokens of each request come one a step (as decoding would bring them)."""
    rng = np.random.default_rng(seed)
    waiting = list(requests)
    live = []          # [rid, ids, pos, k]
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, ids = waiting.pop(0)
            live.append([rid, list(ids), 0, int(rng.integers(0, 5))])
        entries, ends = [], []
        for item in live:
            rid, ids, pos, k = item
            if len(live) > 1 and rng.random() < 0.2:
                continue                                # left out of this step, goes on later
            if pos >= len(ids) - decode_tail:
                n = 1
            else:
                n = min(prefill_sizes[k % len(prefill_sizes)], len(ids) - decode_tail - pos)
                item[3] += 1
            entries.append({"id": rid, "tokens": ids[pos:pos + n], "want": list(range(n))})
            item[2] = pos + n
            if item[2] >= len(ids):
                ends.append(rid)
        live = [it for it in live if it[0] not in ends]
        if entries or ends:
            steps.append({"step": len(steps), "entries": entries, "end": ends})
    return steps


def max_live_tokens(steps, round_to=64):
    """The --max-tokens a trace needs: most tokens live requests hold, each rounded up."""
    held, worst = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return worst


def replay(session, steps):
    """Run a trace on a TraceSession; returns {rid: [T, V] array} assembled from wanted rows."""
    got = {}
    for s in steps:
        out = session.run_step(s)
        r = 0
        for e in s["entries"]:
            for _ in e.get("want", []):
                got.setdefault(e["id"], []).append(out[r])
                r += 1
    return {rid: np.stack(rows) for rid, rows in got.items()}


# bfloat16 bounds relative to the logits' root mean square: the largest error and the rms error (about
# four bfloat16 roundings of 2^-9 each end to end)
BF16_MAX_OF_RMS, BF16_RMS_OF_RMS = 4e-2, 2.0 ** -7


def bf16_token_slack(plain_row):
    """How far below the plain maximum a token picked in bfloat16 may lie: two logits, each off by the
    largest error the bfloat16 bound allows."""
    return 2 * BF16_MAX_OF_RMS * float(np.sqrt((np.asarray(plain_row) ** 2).mean()))


def check_against_plain(model: TinyModel, got, requests, dtype, what="", rows=None):
    """32-bit: every logit within ATOL of the plain model's.  bfloat16: the largest error within 4 % of
    the logits' rms and the rms error within 2^-7 of it, at every size (the logits' rms is 0.16 to 0.2 on
    the tiny models and 0.55 to 0.8 at the benchmark models' layer sizes).  ``rows[rid]`` names the
    positions that ``got[rid]`` holds when it does not hold all."""
    for rid, ids in requests:
        ref = model.plain_logits(ids)
        if rows is not None:
            ref = ref[rows[rid]]
        out = got[rid]
        assert out.shape == ref.shape, f"{what} {rid}: shape {out.shape} vs {ref.shape}"
        err = np.abs(out.astype(np.float64) - ref)
        worst = np.unravel_index(np.argmax(err), err.shape)
        if dtype == "float32":
            atol = ATOL[dtype]
        else:
            rms = float(np.sqrt((model.plain_logits(ids) ** 2).mean()))
            atol = BF16_MAX_OF_RMS * rms
            rms_err = float(np.sqrt((err ** 2).mean()))
            assert rms_err <= BF16_RMS_OF_RMS * rms, (f"{what} request {rid} ({dtype}): rms error {rms_err:.3e} > "
                                                      f"2^-7 of the logits' rms {rms:.3e}")
        assert err.max() <= atol, (f"{what} request {rid} ({dtype}): max abs error {err.max():.3e} > {atol:.1e}; "
                                   f"first bad position {int(np.argmax(err.max(axis=1) > atol))}, worst at "
                                   f"position {worst[0]} token {worst[1]}")
