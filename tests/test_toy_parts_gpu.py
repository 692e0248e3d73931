"""A toy architecture defined here, in the test: a mixer with state of its own (a running mean
per request, kept in a state slot), registered, built from a model folder and stepped through
the engine -- without a change to the framework's files.  Its run order also names a layer
twice and lets a layer read another layer's cache.  It is no model of anyone's; it shows that
the parts, the registries, the cache slots and the step function carry more than GPT-2."""
import json
import math
import os
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import helpers
import plain_gpt2 as P

pytestmark = pytest.mark.gpu

E, H, D, V, NPOS, INNER = 64, 4, 16, 300, 96, 96
EPS = 1e-5


# ------------------------------------------------------------------ the toy mixer (test-side code)
@dataclass(frozen=True)
class RunningMeanSpec:
    kind: str
    width: int


def _register_once():
    from deliverance_amd.config import (AttentionSpec, DenseFeedForwardSpec, LayerCall, LayerSpec, ModelConfig,
                                        NormSpec, PositionSpec)
    from deliverance_amd.kernels import ops
    from deliverance_amd.parts import Mixer, StateNeed, register_mixer, to_matrix
    from deliverance_amd.registry import Architecture, ModelSupport
    from deliverance_amd.weights import TensorDecl
    if "toyrunningmeanlm" in ModelSupport._by_name:
        return

    class RunningMean(Mixer):
        """y_t = W . mean(h_0 .. h_t).  State per request: the sum so far (width floats) and the count.
        Everything it reads about the step lies on the device (the rows' sequences, the portions' first
        rows, the sequences' state slots), so a decode step with this mixer is recorded and replayed
        like any other."""
        graph_safe = True

        def __init__(self, spec, params, dtype, device):
            self.width = spec.width
            self.weight = to_matrix(params["weight"], dtype, device)

        def cache_need(self):
            return StateNeed(self.width + 1)

        def forward(self, ctx, h, x, call):
            state = ctx.cache.state[call.cache]                       # [slots, width + 1], float32
            N, Wd = h.shape[0], self.width
            before = ops.state_gather(state, ctx.state_slots, ctx.seq_of_token, ctx.buf("toy_before", N, Wd + 1, torch.float32))
            first = ctx.q_start.long()[ctx.seq_of_token[:N].long()]   # the first row of each row's portion
            c = torch.cumsum(h.float(), dim=0)
            base = torch.where((first > 0)[:, None], c[(first - 1).clamp(min=0)], torch.zeros_like(c))
            after = ctx.buf("toy_after", N, Wd + 1, torch.float32)
            after[:, :Wd] = c - base + before[:, :Wd]
            after[:, Wd] = before[:, Wd] + (torch.arange(N, device=h.device) - first + 1).float()
            means = ctx.buf("toy_means", N, Wd, ctx.dtype)
            means.copy_(after[:, :Wd] / after[:, Wd:])
            if call.write:                                            # what a portion's last row leaves is the state
                ops.state_scatter(state, ctx.state_slots, ctx.q_start, after, ctx.n_seqs)
            ops.linear(means, self.weight, None, x, accumulate=True)

    register_mixer("toy_running_mean", RunningMean)

    def read_config(d):
        norm = NormSpec("layernorm", E, EPS)
        attn = AttentionSpec("attention", E, H, H, D, 1 / math.sqrt(D))
        ff = DenseFeedForwardSpec("dense", E, INNER, "gelu_new")
        layers = (LayerSpec(attn, ff, norm, None, norm, None, "l0."),
                  LayerSpec(RunningMeanSpec("toy_running_mean", E), None, norm, None, None, None, "l1."),
                  LayerSpec(attn, ff, norm, None, norm, None, "l2."))
        # layer 0 runs twice (its second run has a cache slot of its own); layer 2 reads the keys and
        # values that layer 0's first run wrote, and writes none
        schedule = (LayerCall(0, 0, True), LayerCall(1, 1, True), LayerCall(0, 2, True), LayerCall(2, 0, False))
        return ModelConfig("ToyRunningMeanLM", V, E, NPOS, layers, schedule, PositionSpec("learned", NPOS), norm,
                           True, None, (), raw=dict(d))

    def declare(mc):
        out = [TensorDecl("emb.weight", (V, E)), TensorDecl("pos.weight", (NPOS, E), std=0.01),
               TensorDecl("final.weight", (E,), "ones_plus_normal", 0.1), TensorDecl("final.bias", (E,))]
        for p in ("l0.", "l2."):
            out += [TensorDecl(p + "n1.weight", (E,), "ones_plus_normal", 0.1), TensorDecl(p + "n1.bias", (E,)),
                    TensorDecl(p + "qkv.weight", (3 * E, E), std=0.1), TensorDecl(p + "qkv.bias", (3 * E,)),
                    TensorDecl(p + "o.weight", (E, E), std=0.1), TensorDecl(p + "o.bias", (E,)),
                    TensorDecl(p + "n2.weight", (E,), "ones_plus_normal", 0.1), TensorDecl(p + "n2.bias", (E,)),
                    TensorDecl(p + "fc.weight", (INNER, E), std=0.1), TensorDecl(p + "fc.bias", (INNER,)),
                    TensorDecl(p + "pr.weight", (E, INNER), std=0.1), TensorDecl(p + "pr.bias", (E,))]
        out += [TensorDecl("l1.n1.weight", (E,), "ones_plus_normal", 0.1), TensorDecl("l1.n1.bias", (E,)),
                TensorDecl("l1.mix.weight", (E, E), std=0.1)]
        return out

    def bind(mc, t):
        def attn_layer(p):
            return {"pre_mixer_norm": {"weight": t[p + "n1.weight"], "bias": t[p + "n1.bias"]},
                    "mixer": {"qkv_weight": t[p + "qkv.weight"], "qkv_bias": t[p + "qkv.bias"],
                              "out_weight": t[p + "o.weight"], "out_bias": t[p + "o.bias"]},
                    "pre_ff_norm": {"weight": t[p + "n2.weight"], "bias": t[p + "n2.bias"]},
                    "feed_forward": {"fc_weight": t[p + "fc.weight"], "fc_bias": t[p + "fc.bias"],
                                     "proj_weight": t[p + "pr.weight"], "proj_bias": t[p + "pr.bias"]}}
        toy = {"pre_mixer_norm": {"weight": t["l1.n1.weight"], "bias": t["l1.n1.bias"]},
               "mixer": {"weight": t["l1.mix.weight"]}}
        return {"embed": {"tokens": t["emb.weight"], "positions": {"table": t["pos.weight"]}},
                "layers": [attn_layer("l0."), toy, attn_layer("l2.")],
                "final_norm": {"weight": t["final.weight"], "bias": t["final.bias"]},
                "head": {"weight": t["emb.weight"]}}

    ModelSupport.add_model(Architecture("ToyRunningMeanLM", read_config, declare, bind))


# ------------------------------------------------------------------ the same model, plainly
def plain_toy(W, ids):
    T = len(ids)
    x = P.embed(ids, np.arange(T), W["emb.weight"], W["pos.weight"])

    def qkv(p, a):
        z = a @ W[p + "qkv.weight"].T + W[p + "qkv.bias"]
        return z[:, :E], z[:, E:2 * E], z[:, 2 * E:]

    def attn_layer(p, x, kv_from=None):
        a = P.layer_norm(x, W[p + "n1.weight"], W[p + "n1.bias"], EPS)
        q, k, v = qkv(p, a)
        if kv_from is not None:
            k, v = kv_from
        o = P.causal_attention(q, k, v, H, 1 / math.sqrt(D))
        x = x + o @ W[p + "o.weight"].T + W[p + "o.bias"]
        m = P.layer_norm(x, W[p + "n2.weight"], W[p + "n2.bias"], EPS)
        x = x + P.gelu_tanh(m @ W[p + "fc.weight"].T + W[p + "fc.bias"]) @ W[p + "pr.weight"].T + W[p + "pr.bias"]
        return x, (k, v)

    x, kv0 = attn_layer("l0.", x)
    a = P.layer_norm(x, W["l1.n1.weight"], W["l1.n1.bias"], EPS)
    means = np.cumsum(a, axis=0) / np.arange(1, T + 1)[:, None]
    x = x + means @ W["l1.mix.weight"].T
    x, _ = attn_layer("l0.", x)                      # the same layer, run a second time
    x, _ = attn_layer("l2.", x, kv_from=kv0)         # reads what the first run of layer 0 cached
    e = P.layer_norm(x, W["final.weight"], W["final.bias"], EPS)
    return e @ W["emb.weight"].T


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    _register_once()
    from deliverance_amd.random_model import random_model
    folder = str(tmp_path_factory.mktemp("toy"))
    random_model(folder, {"architectures": ["ToyRunningMeanLM"], "note": "test-only"}, seed=3)
    return folder


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_is_registered_built_and_stepped(toy_folder, dtype):
    from deliverance_amd.parts import KVNeed, StateNeed
    _, W = P.read_model_folder(toy_folder)
    s = helpers.trace_session(toy_folder, dtype, 256, poison_freed=True)
    needs = s.model.cache_needs()
    assert isinstance(needs[0], KVNeed) and isinstance(needs[1], StateNeed) and isinstance(needs[2], KVNeed)
    assert needs[1].elems == E + 1 and set(s.cache.state) == {1}
    rng = np.random.default_rng(0)
    reqs = [(f"t{i}", [int(t) for t in rng.integers(0, V, size=n)]) for i, n in enumerate((40, 9, 70, 23))]
    tol = {"float32": 2e-5, "bfloat16": 6e-2}[dtype]
    ref = {rid: plain_toy(W, ids) for rid, ids in reqs}
    for name, steps in (("whole", sum((helpers.trace_whole(r, ids) for r, ids in reqs), [])),
                        ("portions", sum((helpers.trace_portions(r, ids) for r, ids in reqs), [])),
                        ("bulk+single", sum((helpers.trace_bulk_then_single(r, ids, 16) for r, ids in reqs), [])),
                        ("mixed", helpers.trace_mixed(reqs, seed=5))):
        for i, st in enumerate(steps):
            st["step"] = i
        got = helpers.replay(s, steps)
        for rid, ids in reqs:
            err = np.abs(got[rid] - ref[rid]).max()
            assert err < tol, f"{name} {rid}: {err}"
        s.cache.manager.check()
        assert s.cache.manager.live() == []
    # a state slot is handed to the next request zeroed: the same request twice gives the same logits
    a = helpers.replay(s, helpers.trace_whole("again", reqs[0][1]))["again"]
    b = helpers.replay(s, helpers.trace_whole("again", reqs[0][1]))["again"]
    assert np.array_equal(a, b)


@pytest.mark.needs_device
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_decodes_from_recorded_graphs(toy_folder, dtype):
    """The mixer with state inside recorded decode steps: batches of 5, 4, 3, 2, 1 padded to buckets and
    replayed (every bucket several times, with eager prompt steps of later requests between the replays),
    each step's logits against the plain model."""
    from test_engine_paths_gpu import decode_trace
    _, W = P.read_model_folder(toy_folder)
    s = helpers.trace_session(toy_folder, dtype, 512, poison_freed=True, use_graphs=True, sample=True)
    assert s.model.graph_safe and s.runner.use_graphs
    rng = np.random.default_rng(4)
    tol = {"float32": 2e-5, "bfloat16": 6e-2}[dtype]
    for round_ in range(2):                     # the second round replays the graphs that the first recorded
        reqs = [(f"g{round_}{i}", [int(t) for t in rng.integers(0, V, size=n)]) for i, n in enumerate((30, 17, 44, 9, 25))]
        got = helpers.replay(s, decode_trace(reqs, [5, 9, 14, 3, 20]))
        for rid, ids in reqs:
            err = np.abs(got[rid] - plain_toy(W, ids)).max()
            assert err < tol, f"round {round_} {rid}: {err}"
        s.cache.manager.check()
        assert s.cache.manager.live() == []
    assert len(s.runner._graphs) >= 3


@pytest.mark.needs_device
def test_toy_architecture_generates_through_the_entry_point(toy_folder):
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    _, W = P.read_model_folder(toy_folder)
    model = AutoModelForCausalLM.from_pretrained(toy_folder, dtype="float32", max_cached_tokens=512, max_num_seqs=4)
    rng = np.random.default_rng(1)
    prompts = [[int(t) for t in rng.integers(0, V, size=n)] for n in (7, 20)]
    outs = model.generate(prompts, GeneratorParameters(max_tokens=6))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for _ in range(6):
            ids.append(int(np.argmax(plain_toy(W, ids)[-1])))
        assert out.generated_tokens == ids[len(prompt):]


def test_run_order_mistakes_are_refused(toy_folder):
    from deliverance_amd.config import LayerCall
    from deliverance_amd.models.causal_lm import CausalLM
    from deliverance_amd.registry import ModelSupport, read_config_json
    from deliverance_amd.weights import load_declared
    import dataclasses
    arch = ModelSupport.detect(read_config_json(toy_folder))
    mc = arch.read_config(read_config_json(toy_folder))
    t = load_declared(toy_folder, arch.declare_tensors(mc))
    bad = dataclasses.replace(mc, schedule=(LayerCall(0, 0, True), LayerCall(2, 0, True)))
    with pytest.raises(ValueError, match="written by two"):
        CausalLM(bad, arch.bind_tensors(bad, t), torch.float32, helpers.DEVICE).cache_needs()
    bad = dataclasses.replace(mc, schedule=(LayerCall(0, 0, True), LayerCall(2, 5, False)))
    with pytest.raises(ValueError, match="nothing writes"):
        CausalLM(bad, arch.bind_tensors(bad, t), torch.float32, helpers.DEVICE).cache_needs()
    bad = dataclasses.replace(mc, schedule=(LayerCall(0, 0, True), LayerCall(7, 1, True)))
    with pytest.raises(ValueError, match="run order names layer 7"):
        CausalLM(bad, arch.bind_tensors(bad, t), torch.float32, helpers.DEVICE)
