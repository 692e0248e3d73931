"""Pins for the plain implementation beside the reference's text (no GPU): vectors the
reference's own tests hold, special cases that reduce to a library routine, invariants.  Each
is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import helpers
import plain_gpt2 as P


def test_layernorm_vector_of_the_reference():
    # core/src/test/java/io/teknek/deliverance/geneator/LayerNormTest.java:40,51,77,88 (eps 1e-5, no affine)
    x = np.array([[-1.1151, 0.1490, -1.0923, -1.4551, 1.3358, 0.3075, 0.6278]])
    want = np.array([[-0.9635, 0.3355, -0.9401, -1.3129, 1.5551, 0.4984, 0.8275]])
    got = P.layer_norm(x, np.ones(7), np.zeros(7), 1e-5)
    assert np.abs(got - want).max() < 1e-4        # an unbiased variance would give -0.892 in column 0


def test_layernorm_is_the_library_routine():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(5, 33)) * 3 + 1
    w, b = rng.normal(size=33), rng.normal(size=33)
    for eps in (1e-5, 1e-1):                       # a large eps shows eps outside the root or ignored
        want = F.layer_norm(torch.tensor(x), (33,), torch.tensor(w), torch.tensor(b), eps).numpy()
        assert np.abs(P.layer_norm(x, w, b, eps) - want).max() < 1e-12


def test_gelu_forms():
    x = np.linspace(-6, 6, 241)
    assert np.abs(P.gelu_erf(x) - F.gelu(torch.tensor(x)).numpy()).max() < 1e-12
    assert np.abs(P.gelu_tanh(x) - F.gelu(torch.tensor(x), approximate="tanh").numpy()).max() < 1e-12
    assert np.abs(P.gelu_erf(x) - P.gelu_tanh(x)).max() > 1e-4          # the two forms are told apart
    # the reference's polynomial erf (math/.../ActivationFunction.java:24-31) stays within 1e-6 of the exact form
    assert np.abs(P.gelu_erf_reference_polynomial(x) - P.gelu_erf(x)).max() < 1e-6
    assert P.gelu_erf(np.array([0.0]))[0] == 0 and abs(P.gelu_erf(np.array([10.0]))[0] - 10) < 1e-9


def test_attention_reduces_to_the_library_routine():
    rng = np.random.default_rng(1)
    T, H, D = 9, 3, 16
    q, k, v = (rng.normal(size=(T, H * D)) for _ in range(3))
    scale = 0.37                                    # not 1/sqrt(D): shows a scale applied twice or not at all
    got = P.causal_attention(q, k, v, H, scale)

    def heads(a):
        return torch.tensor(a).reshape(T, H, D).transpose(0, 1)[None]
    want = F.scaled_dot_product_attention(heads(q), heads(k), heads(v), is_causal=True, scale=scale)[0]
    want = want.transpose(0, 1).reshape(T, H * D).numpy()
    assert np.abs(got - want).max() < 1e-12
    # one head, no mask to speak of (last row sees all): plain softmax(q k^T) v
    q1, k1, v1 = (rng.normal(size=(T, D)) for _ in range(3))
    last = P.causal_attention(q1, k1, v1, 1, 1.0)[-1]
    w = torch.softmax(torch.tensor(k1 @ q1[-1]), 0).numpy()
    assert np.abs(last - w @ v1).max() < 1e-12


def test_attention_invariants():
    rng = np.random.default_rng(2)
    T, H, D = 12, 2, 16
    q, k, v = (rng.normal(size=(T, H * D)) for _ in range(3))
    out = P.causal_attention(q, k, v, H, 0.25)
    # the first token's output is its own value
    assert np.abs(out[0] - v[0]).max() < 1e-12
    # a token is untouched by later tokens
    k2, v2 = k.copy(), v.copy()
    k2[7:] += 5.0; v2[7:] -= 3.0
    assert np.abs(P.causal_attention(q, k2, v2, H, 0.25)[:7] - out[:7]).max() == 0
    assert np.abs(P.causal_attention(q, k2, v2, H, 0.25)[7:] - out[7:]).max() > 1e-3
    # a window of w keys: tokens before position w are unchanged, later ones lose the far keys
    win = P.causal_attention(q, k, v, H, 0.25, window=4)
    assert np.abs(win[:4] - out[:4]).max() == 0 and np.abs(win[4:] - out[4:]).max() > 1e-6
    assert np.abs(win[9] - P.causal_attention(q[6:10], k[6:10], v[6:10], H, 0.25)[-1]).max() < 1e-12
    # `past`: the last rows of a longer sequence
    assert np.abs(P.causal_attention(q[8:], k, v, H, 0.25, past=8) - out[8:]).max() == 0
    # fewer key heads: both query heads of a group read the same keys
    kk, vv = k[:, :D], v[:, :D]
    g = P.causal_attention(q, kk, vv, H, 0.25, n_kv_head=1)
    assert np.abs(g[:, D:] - P.causal_attention(q[:, D:], kk, vv, 1, 0.25)).max() < 1e-12


def test_conv1d_is_addmm_on_the_stored_layout():
    rng = np.random.default_rng(3)
    x, w, b = rng.normal(size=(4, 6)), rng.normal(size=(6, 10)), rng.normal(size=10)
    want = torch.addmm(torch.tensor(b), torch.tensor(x), torch.tensor(w)).numpy()
    assert np.abs(P.conv1d(x, w, b) - want).max() < 1e-12
    # the reference's convention r[i,j] = sum_k a[i,k] b[j,k] on the transposed weight
    # (tensor/.../operations/NaiveTensorOperations.java:86-91)
    wt = w.T
    r = np.array([[sum(x[i, kk] * wt[j, kk] for kk in range(6)) for j in range(10)] for i in range(4)]) + b
    assert np.abs(P.conv1d(x, w, b) - r).max() < 1e-12


def test_block_structure(model_a):
    cfg, W = model_a.plain_cfg, model_a.W
    rng = np.random.default_rng(4)
    x = rng.normal(size=(6, cfg["n_embd"]))
    # zero output projections (weights and biases): the block is the identity
    Z = dict(W)
    for k in ("h.0.attn.c_proj.weight", "h.0.attn.c_proj.bias", "h.0.mlp.c_proj.weight", "h.0.mlp.c_proj.bias"):
        Z[k] = np.zeros_like(W[k])
    assert np.abs(P.block(x, Z, 0, cfg) - x).max() == 0
    # zero attention projection only: x + MLP(LN2(x)), so the second norm reads the stream, not LN1's output
    Z2 = dict(W)
    Z2["h.0.attn.c_proj.weight"] = np.zeros_like(W["h.0.attn.c_proj.weight"])
    Z2["h.0.attn.c_proj.bias"] = np.zeros_like(W["h.0.attn.c_proj.bias"])
    m = P.layer_norm(x, W["h.0.ln_2.weight"], W["h.0.ln_2.bias"], cfg["layer_norm_epsilon"])
    assert np.abs(P.block(x, Z2, 0, cfg) - (x + P.mlp_block(m, W, 0, cfg["activation_function"]))).max() < 1e-12


def test_fused_projection_is_three_projections_in_q_k_v_order(model_b):
    """The plain attention block is its parts put together: the fused projection's columns taken as
    thirds q | k | v (core/src/main/java/io/teknek/deliverance/model/gpt2/Gpt2Model.java:81-82 slices
    c_attn in that order), attention, output projection.  Parity unpinned: the reference holds no vector
    for GPT-2's attention block, so the ORDER of the thirds rests on reading those two lines; what this
    test can catch is a plain block whose parts are not wired as its own functions say (a swapped k and
    v shows: the result below changes by far more than rounding), and the engine's order is held to the
    plain model's by every replay test."""
    cfg, W = model_b.plain_cfg, model_b.W
    E, H = cfg["n_embd"], cfg["n_head"]
    rng = np.random.default_rng(5)
    a = rng.normal(size=(7, E))
    w, b = W["h.1.attn.c_attn.weight"], W["h.1.attn.c_attn.bias"]
    q, k, v = (a @ w[:, i * E:(i + 1) * E] + b[i * E:(i + 1) * E] for i in range(3))
    scale = 1 / math.sqrt(E // H) / 2                 # layer 1 with scale_attn_by_inverse_layer_idx
    o = P.causal_attention(q, k, v, H, scale)
    want = o @ W["h.1.attn.c_proj.weight"] + W["h.1.attn.c_proj.bias"]
    assert np.abs(P.attention_block(a, W, 1, H, scale) - want).max() < 1e-12
    swapped = P.causal_attention(q, v, k, H, scale) @ W["h.1.attn.c_proj.weight"] + W["h.1.attn.c_proj.bias"]
    assert np.abs(swapped - want).max() > 1e-3


def test_whole_model_properties(model_a, model_b):
    for m in (model_a, model_b):
        ids = m.prompt(20)
        lg = P.forward_logits(m.plain_cfg, m.W, ids)
        assert lg.shape == (20, m.cfg["vocab_size"]) and np.isfinite(lg).all()
        # prefix property: logits at position t do not depend on later tokens
        assert np.abs(P.forward_logits(m.plain_cfg, m.W, ids[:11]) - lg[:11]).max() < 1e-12
        # positions are absolute: the same tokens one place later give other logits
        shifted = P.forward_logits(m.plain_cfg, m.W, [ids[0]] + ids)[1:]
        assert np.abs(shifted - lg).max() > 1e-4
        # tied head: scaling the table changes both ends
        W2 = dict(m.W); W2["wte.weight"] = m.W["wte.weight"] * 1.5
        assert np.abs(P.forward_logits(m.plain_cfg, W2, ids) - 1.5 * lg).max() > 1e-3
    # every prompt length 1..n is finite (HfModelTesterMixinPort.java:28-97)
    for n in range(1, 6):
        assert np.isfinite(P.forward_logits(model_b.plain_cfg, model_b.W, model_b.prompt(n))).all()
    # float32 arithmetic agrees with float64 to rounding
    c32, W32 = P.read_model_folder(model_a.folder, np.float32)
    ids = model_a.prompt(17)
    assert np.abs(P.forward_logits(c32, W32, ids) - model_a.plain_logits(ids)).max() < 2e-5


def test_config_b_options_matter(model_b):
    ids = model_b.prompt(12)
    base = model_b.plain_logits(ids)
    for key, val in (("scale_attn_by_inverse_layer_idx", False), ("activation_function", "gelu_new"),
                     ("layer_norm_epsilon", 1e-2)):
        cfg = dict(model_b.plain_cfg); cfg[key] = val
        assert np.abs(P.forward_logits(cfg, model_b.W, ids) - base).max() > 1e-5, key


def test_java_random_and_sampler_vectors():
    r = P.JavaRandom(42)
    assert abs(r.next_float() - 0.7275637) < 1e-6          # new java.util.Random(42).nextFloat()
    # core/src/test/java/io/teknek/deliverance/model/TopKSamplerTest.java:13-54
    assert P.top_k_candidate_count(64.0, 262144) == 64
    assert P.top_k_candidate_count(0.10, 100) == 90
    logits = [5.0, 4.0, 3.0, 2.0, 1.0]
    assert P.sample_top_k_top_p(logits, 1.0, 2.0, 0.95, None, 0.99) == 1
    assert P.sample_top_k_top_p(logits, 1.0, 2.0, 0.95, None, 0.60) == 0
    assert P.sample_top_k_top_p(logits, 1.0, 2.0, 0.95, 1.0, 0.60) == 1
    for bad in (0.0, 1.01):
        with pytest.raises(ValueError):
            P.sample_top_k_top_p([2.0, 1.0], 1.0, None, None, bad, 0.5)
    with pytest.raises(ValueError):
        P.sample_top_k_top_p([2.0, 1.0], 1.0, None, None, 1.0, 0.5)
    # ties keep index order (a stable sort): with equal logits and u just past 1/3 the second token is picked
    assert P.sample_top_k_top_p([1.0, 1.0, 1.0], 1.0, None, None, None, 0.34) == 1
    # the nucleus keeps the token that crosses p
    probs = np.exp(np.array(logits) - 5); probs /= probs.sum()
    assert P.sample_top_k_top_p(logits, 1.0, None, float(probs[0] + 0.01), None, 0.999) == 1
