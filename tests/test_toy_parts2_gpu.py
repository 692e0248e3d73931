"""A second toy architecture defined in the test: a position encoding that acts on queries
and keys (a rotation of pairs by an angle that grows with the position), attention with fewer
key heads than query heads and a window in one layer, one key head and no window in the other
(two cache groups with pages of their own; the windowed group gives pages back while a request
runs), a feed-forward with routing (two experts, the larger router logit wins) in one layer
and the framework's dense one in the other, and a head that is not tied to the embedding.
All of it is registered, built from a model folder and stepped without a change to the
framework's files.  It is no model of anyone's."""
import math
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import helpers
import plain_gpt2 as P

pytestmark = pytest.mark.gpu

E, V, NPOS = 96, 257, 160
H0, HKV0, D0, WINDOW, BASE = 6, 2, 16, 24, 100.0     # layer 0: grouped heads, a window, rotated pairs
H1, HKV1, D1 = 3, 1, 32                              # layer 1: one key head, every earlier key
INNER0, INNER_X, N_EXPERTS = 80, 48, 2
EPS = 1e-6
LOGIT_MULT = 2.5     # the logits are divided by it (an architecture's constant)
MARGIN = 0.05        # rows whose router logits lie closer than this are left out of the bfloat16 comparison


@dataclass(frozen=True)
class RoutedSpec:
    kind: str
    width: int
    inner: int
    n_experts: int


def _register_once():
    from deliverance_amd.config import (AttentionSpec, DenseFeedForwardSpec, LayerCall, LayerSpec, ModelConfig,
                                        NormSpec, PositionSpec)
    from deliverance_amd.parts import (FeedForward, PositionEncoding, register_feed_forward, register_position,
                                       to_matrix)
    from deliverance_amd.registry import Architecture, ModelSupport
    from deliverance_amd.weights import TensorDecl
    if "toywindowroutelm" in ModelSupport._by_name:
        return

    class PairRotation(PositionEncoding):
        """q and k: the pair (2i, 2i+1) of every head is turned by position * base^(-i / (D/2))."""

        def __init__(self, spec, params, dtype, device):
            self.base = dict(spec.params)["base"]

        def apply_qk(self, ctx, qkv, n_heads, n_kv_heads, head_dim):
            N, half = qkv.shape[0], head_dim // 2
            inv = self.base ** (-torch.arange(half, device=qkv.device, dtype=torch.float32) / half)
            ang = ctx.positions[:N].float()[:, None] * inv[None, :]
            cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            for first, heads in ((0, n_heads), (n_heads * head_dim, n_kv_heads)):
                block = qkv[:, first:first + heads * head_dim]
                b = block.float().reshape(N, heads, half, 2)
                x0, x1 = b[..., 0], b[..., 1]
                y = torch.stack((x0 * cos - x1 * sin, x0 * sin + x1 * cos), dim=-1)
                block.copy_(y.reshape(N, heads * head_dim).to(qkv.dtype))

    class Routed(FeedForward):
        """x += p * expert_e(h), e the expert with the larger router logit, p its softmax weight (32-bit)."""

        def __init__(self, spec, params, dtype, device):
            self.n = spec.n_experts
            self.router = params["router"].to(device=device, dtype=torch.float32)
            self.fc = [to_matrix(params[f"fc{e}"], dtype, device) for e in range(self.n)]
            self.pr = [to_matrix(params[f"pr{e}"], dtype, device) for e in range(self.n)]

        def forward(self, ctx, h, x):
            logits = h.float() @ self.router.t()
            best = logits.argmax(dim=1)
            p = torch.softmax(logits, dim=1).gather(1, best[:, None])
            for e in range(self.n):
                rows = (best == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                mid = torch.nn.functional.gelu(h[rows].float() @ self.fc[e].float().t(), approximate="tanh").to(h.dtype)
                x[rows] += p[rows] * (mid.float() @ self.pr[e].float().t())

    register_position("toy_pair_rotation", PairRotation)
    register_feed_forward("toy_routed", Routed)

    def read_config(d):
        norm = NormSpec("layernorm", E, EPS)
        a0 = AttentionSpec("attention", E, H0, HKV0, D0, 1 / math.sqrt(D0), window=WINDOW,
                           position=PositionSpec("toy_pair_rotation", NPOS, (("base", BASE),)))
        a1 = AttentionSpec("attention", E, H1, HKV1, D1, 1 / math.sqrt(D1), qkv_bias=False, out_bias=False)
        layers = (LayerSpec(a0, DenseFeedForwardSpec("dense", E, INNER0, "relu"), norm, None, norm, None, "l0."),
                  LayerSpec(a1, RoutedSpec("toy_routed", E, INNER_X, N_EXPERTS), norm, None, norm, None, "l1."))
        return ModelConfig("ToyWindowRouteLM", V, E, NPOS, layers, (LayerCall(0, 0, True), LayerCall(1, 1, True)),
                           PositionSpec("none"), norm, False, None, (), raw=dict(d), logit_multiplier=LOGIT_MULT)

    def declare(mc):
        q0, q1 = (H0 + 2 * HKV0) * D0, (H1 + 2 * HKV1) * D1
        out = [TensorDecl("emb.weight", (V, E), std=0.5), TensorDecl("head.weight", (V, E), std=0.1),
               TensorDecl("final.weight", (E,), "ones_plus_normal", 0.1), TensorDecl("final.bias", (E,))]
        for p in ("l0.", "l1."):
            out += [TensorDecl(p + "n1.weight", (E,), "ones_plus_normal", 0.1), TensorDecl(p + "n1.bias", (E,)),
                    TensorDecl(p + "n2.weight", (E,), "ones_plus_normal", 0.1), TensorDecl(p + "n2.bias", (E,))]
        out += [TensorDecl("l0.qkv.weight", (q0, E), std=0.15), TensorDecl("l0.qkv.bias", (q0,)),
                TensorDecl("l0.o.weight", (E, H0 * D0), std=0.1), TensorDecl("l0.o.bias", (E,)),
                TensorDecl("l0.fc.weight", (INNER0, E), std=0.1), TensorDecl("l0.fc.bias", (INNER0,)),
                TensorDecl("l0.pr.weight", (E, INNER0), std=0.1), TensorDecl("l0.pr.bias", (E,)),
                TensorDecl("l1.qkv.weight", (q1, E), std=0.15), TensorDecl("l1.o.weight", (E, H1 * D1), std=0.1),
                TensorDecl("l1.router.weight", (N_EXPERTS, E), std=0.5)]
        for e in range(N_EXPERTS):
            out += [TensorDecl(f"l1.x{e}.fc.weight", (INNER_X, E), std=0.1),
                    TensorDecl(f"l1.x{e}.pr.weight", (E, INNER_X), std=0.1)]
        return out

    def bind(mc, t):
        def norms(p):
            return {"pre_mixer_norm": {"weight": t[p + "n1.weight"], "bias": t[p + "n1.bias"]},
                    "pre_ff_norm": {"weight": t[p + "n2.weight"], "bias": t[p + "n2.bias"]}}
        l0 = dict(norms("l0."),
                  mixer={"qkv_weight": t["l0.qkv.weight"], "qkv_bias": t["l0.qkv.bias"],
                         "out_weight": t["l0.o.weight"], "out_bias": t["l0.o.bias"], "position": {}},
                  feed_forward={"fc_weight": t["l0.fc.weight"], "fc_bias": t["l0.fc.bias"],
                                "proj_weight": t["l0.pr.weight"], "proj_bias": t["l0.pr.bias"]})
        ff1 = {"router": t["l1.router.weight"]}
        for e in range(N_EXPERTS):
            ff1[f"fc{e}"], ff1[f"pr{e}"] = t[f"l1.x{e}.fc.weight"], t[f"l1.x{e}.pr.weight"]
        l1 = dict(norms("l1."), mixer={"qkv_weight": t["l1.qkv.weight"], "out_weight": t["l1.o.weight"]},
                  feed_forward=ff1)
        return {"embed": {"tokens": t["emb.weight"], "positions": {}}, "layers": [l0, l1],
                "final_norm": {"weight": t["final.weight"], "bias": t["final.bias"]},
                "head": {"weight": t["head.weight"]}}

    ModelSupport.add_model(Architecture("ToyWindowRouteLM", read_config, declare, bind))


# ------------------------------------------------------------------ the same model, plainly
def rotate_pairs(z, n_heads, D, positions):
    half = D // 2
    inv = BASE ** (-np.arange(half) / half)
    ang = positions[:, None] * inv[None, :]
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    b = z.reshape(len(positions), n_heads, half, 2)
    y = np.stack((b[..., 0] * cos - b[..., 1] * sin, b[..., 0] * sin + b[..., 1] * cos), axis=-1)
    return y.reshape(z.shape)


def plain_toy(W, ids):
    """Logits [T, V] and, per row, the distance of the two router logits."""
    T = len(ids)
    pos = np.arange(T, dtype=np.float64)
    x = W["emb.weight"][np.asarray(ids)]
    # layer 0: grouped heads, window, rotated pairs; dense feed-forward with ReLU
    a = P.layer_norm(x, W["l0.n1.weight"], W["l0.n1.bias"], EPS)
    z = a @ W["l0.qkv.weight"].T + W["l0.qkv.bias"]
    q, k, v = z[:, :H0 * D0], z[:, H0 * D0:(H0 + HKV0) * D0], z[:, (H0 + HKV0) * D0:]
    q, k = rotate_pairs(q, H0, D0, pos), rotate_pairs(k, HKV0, D0, pos)
    o = P.causal_attention(q, k, v, H0, 1 / math.sqrt(D0), window=WINDOW, n_kv_head=HKV0)
    x = x + o @ W["l0.o.weight"].T + W["l0.o.bias"]
    m = P.layer_norm(x, W["l0.n2.weight"], W["l0.n2.bias"], EPS)
    x = x + np.maximum(m @ W["l0.fc.weight"].T + W["l0.fc.bias"], 0) @ W["l0.pr.weight"].T + W["l0.pr.bias"]
    # layer 1: one key head, every earlier key, no position; routed feed-forward
    a = P.layer_norm(x, W["l1.n1.weight"], W["l1.n1.bias"], EPS)
    z = a @ W["l1.qkv.weight"].T
    q, k, v = z[:, :H1 * D1], z[:, H1 * D1:(H1 + HKV1) * D1], z[:, (H1 + HKV1) * D1:]
    x = x + P.causal_attention(q, k, v, H1, 1 / math.sqrt(D1), n_kv_head=HKV1) @ W["l1.o.weight"].T
    m = P.layer_norm(x, W["l1.n2.weight"], W["l1.n2.bias"], EPS)
    logits = m @ W["l1.router.weight"].T
    best = logits.argmax(axis=1)
    p = P.softmax_rows(logits)[np.arange(T), best]
    y = np.zeros_like(x)
    for e in range(N_EXPERTS):
        rows = best == e
        y[rows] = P.gelu_tanh(m[rows] @ W[f"l1.x{e}.fc.weight"].T) @ W[f"l1.x{e}.pr.weight"].T
    x = x + p[:, None] * y
    f = P.layer_norm(x, W["final.weight"], W["final.bias"], EPS)
    return f @ W["head.weight"].T / LOGIT_MULT, np.abs(logits[:, 0] - logits[:, 1])


def test_the_plain_rotation_keeps_what_only_distances_decide():
    """Scores of rotated queries and keys depend on the distance of their positions alone: a shift
    of all positions leaves them as they are (a wrong sign in one of the four products would not)."""
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=(5, 2 * D0)), rng.normal(size=(5, 2 * D0))
    pos = np.arange(5, dtype=np.float64)
    s0 = rotate_pairs(q, 2, D0, pos) @ rotate_pairs(k, 2, D0, pos).T
    s1 = rotate_pairs(q, 2, D0, pos + 37) @ rotate_pairs(k, 2, D0, pos + 37).T
    assert np.abs(s0 - s1).max() < 1e-9
    assert np.abs(rotate_pairs(q, 2, D0, np.zeros(5)) - q).max() == 0
    assert np.abs(np.linalg.norm(rotate_pairs(q, 2, D0, pos), axis=1) - np.linalg.norm(q, axis=1)).max() < 1e-12


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    _register_once()
    from deliverance_amd.random_model import random_model
    folder = str(tmp_path_factory.mktemp("toy2"))
    random_model(folder, {"architectures": ["ToyWindowRouteLM"], "note": "test-only"}, seed=11)
    return folder


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_groups_rotation_and_routing_through_the_engine(toy_folder, dtype):
    from deliverance_amd.parts import KVNeed
    _, W = P.read_model_folder(toy_folder)
    s = helpers.trace_session(toy_folder, dtype, 512, poison_freed=True)     # pages that the window has passed are NaN again
    needs = s.model.cache_needs()
    assert needs[0] == KVNeed(HKV0, D0, WINDOW) and needs[1] == KVNeed(HKV1, D1, None)
    assert len(s.cache.groups) == 2                         # pages of their own for the two layers
    rng = np.random.default_rng(0)
    reqs = [(f"t{i}", [int(t) for t in rng.integers(0, V, size=n)]) for i, n in enumerate((150, 9, 70, 41))]
    tol = {"float32": 3e-5, "bfloat16": 8e-2}[dtype]
    ref = {rid: plain_toy(W, ids) for rid, ids in reqs}
    for name, steps in (("whole", sum((helpers.trace_whole(r, ids) for r, ids in reqs), [])),
                        ("portions", sum((helpers.trace_portions(r, ids) for r, ids in reqs), [])),
                        ("bulk+single", sum((helpers.trace_bulk_then_single(r, ids, 32) for r, ids in reqs), [])),
                        ("mixed", helpers.trace_mixed(reqs, seed=5))):
        for i, st in enumerate(steps):
            st["step"] = i
        got = helpers.replay(s, steps)
        for rid, ids in reqs:
            want, margin = ref[rid]
            rows = np.ones(len(ids), bool) if dtype == "float32" else margin > MARGIN
            assert rows.sum() > 0.8 * len(ids)
            err = np.abs(got[rid] - want)[rows].max()
            assert err < tol, f"{name} {rid}: {err}"
        s.cache.manager.check()
        assert s.cache.manager.live() == []
    # while a long request runs, the windowed group holds only the pages its window still reaches
    ids = reqs[0][1]
    st = helpers.trace_portions("w", ids, (50, 1, 1, 30, 1))
    st[-1]["end"] = []
    helpers.replay(s, st)
    page = s.cache.page_size
    held = [sum(1 for p in s.cache.manager.table("w", g) if p >= 0) for g in range(2)]
    by_window = [g for g in range(2) if s.cache.groups[g].window is not None][0]
    assert held[1 - by_window] == -(-len(ids) // page)
    assert held[by_window] <= (WINDOW + page - 1) // page + 1 < held[1 - by_window]
    s.cache.manager.close("w")
    assert s.cache.manager.live() == []


@pytest.mark.needs_device
def test_generation_with_the_toy_parts(toy_folder):
    from deliverance_amd import AutoModelForCausalLM, GeneratorParameters
    _, W = P.read_model_folder(toy_folder)
    model = AutoModelForCausalLM.from_pretrained(toy_folder, dtype="float32", max_cached_tokens=1024, max_num_seqs=4)
    assert not model.runner.use_graphs                       # the routed feed-forward reads sizes on the host
    rng = np.random.default_rng(1)
    prompts = [[int(t) for t in rng.integers(0, V, size=n)] for n in (7, 40, 3)]
    outs = model.generate(prompts, GeneratorParameters(max_tokens=30))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for _ in range(30):
            ids.append(int(np.argmax(plain_toy(W, ids)[0][-1])))
        assert out.generated_tokens == ids[len(prompt):]
