"""A plain, slow GPT-2 in NumPy: whole sequences, no cache, one function per part.

Written from the reference's formulas (paths are relative to the reference checkout); it
shares no code with ``deliverance_amd``.  It reads a model folder with the ``safetensors``
package (not with the engine's own reader) and computes in float64 unless told otherwise,
so that it can serve as ground truth for the engine's 32-bit path.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


# --------------------------------------------------------------------------- reading
def read_model_folder(folder, dtype=np.float64):
    """config.json as a dict, tensors as NumPy arrays of ``dtype`` (names with an optional
    ``transformer.`` prefix removed, as the reference addresses them without it:
    core/src/main/java/io/teknek/deliverance/model/gpt2/Gpt2Model.java:37-38,78-79)."""
    import torch
    from safetensors import safe_open
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            key = name[len("transformer."):] if name.startswith("transformer.") else name
            tensors[key] = t.to(torch.float64).numpy().astype(dtype)
    return cfg, tensors


# --------------------------------------------------------------------------- parts
def embed(ids, positions, wte, wpe):
    """x[t] = wte[id_t] + wpe[pos_t]  (core/.../model/gpt2/Gpt2Model.java:42-48)."""
    return wte[np.asarray(ids)] + wpe[np.asarray(positions)]


def layer_norm(x, weight, bias, eps):
    """Per row: mean, biased variance, 1/sqrt(var+eps), times weight plus bias
    (core/.../generator/LayerNorm.java:127-150).  The reference forms the variance as
    E[x^2]-mean^2 in one pass; this is the same quantity computed from centred values."""
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    inv = 1.0 / np.sqrt(var + eps)
    y = (x - mean) * inv * weight
    return y if bias is None else y + bias


def gelu_erf(x):
    """0.5 x (1 + erf(x / sqrt 2))  (math/src/main/java/io/teknek/deliverance/math/
    ActivationFunction.java:16); exact erf instead of the reference's polynomial
    (ActivationFunction.java:24-31), which differs by about 1.5e-7."""
    erf = np.vectorize(math.erf, otypes=[np.float64])
    return (0.5 * x * (1.0 + erf(np.asarray(x, dtype=np.float64) / math.sqrt(2.0)))).astype(x.dtype)


def gelu_tanh(x):
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))  (ActivationFunction.java:17-19)."""
    return 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def gelu_erf_reference_polynomial(x):
    """The reference's own erf approximation (ActivationFunction.java:24-31), kept to show
    how far it is from the exact form."""
    x = np.asarray(x, dtype=np.float64)
    z = x / math.sqrt(2.0)
    ax = np.abs(z)
    t = 1.0 / (1.0 + 0.3275911 * ax)
    y = 1.0 - (((((1.061405429 * t - 1.453152027) * t) + 1.421413741) * t - 0.284496736) * t
               + 0.254829592) * t * np.exp(-ax * ax)
    return 0.5 * x * (1.0 + np.copysign(1.0, z) * y)


ACTIVATIONS = {
    "gelu": gelu_erf,
    "gelu_new": gelu_tanh,
    "gelu_pytorch_tanh": gelu_tanh,
    "relu": lambda x: np.maximum(x, 0),
    "silu": lambda x: x / (1.0 + np.exp(-x)),
}


def conv1d(x, weight, bias):
    """GPT-2 keeps its projections as [in, out]; the reference transposes them at load and
    multiplies with r[i,j] = sum_k a[i,k] b[j,k] (Gpt2Model.java:81-82,93,103,105;
    tensor/src/main/java/io/teknek/deliverance/tensor/operations/
    NaiveTensorOperations.java:86-91), which is x @ weight + bias on the stored layout."""
    return x @ weight + bias


def softmax_rows(s):
    """max, exp(s - max), divide by the sum
    (tensor/.../tensor/VectorTensorMathUtils.java:34-52)."""
    m = s.max(axis=-1, keepdims=True)
    e = np.exp(s - m)
    return e / e.sum(axis=-1, keepdims=True)


def causal_attention(q, k, v, n_head, scale, window=None, n_kv_head=None, past=0):
    """Per head h (columns h*D .. h*D+D-1, core/.../generator/CausalSelfAttention.java:478-479):
    scores q_t . k_j * scale for j <= t only (CausalSelfAttention.java:481-491,512-527),
    softmax, weighted sum of v.  ``window`` w keeps only the last w keys (t-w < j <= t).
    With fewer key heads, query head h reads key head h // (n_head / n_kv_head)
    (tensor/src/test/java/io/teknek/deliverance/tensor/operations/
    TensorOperationsDecodePagedAttentionTest.java:49-57).  ``past``: q holds the last
    len(q) positions of a sequence whose keys are all in k, v."""
    T = q.shape[0]
    D = q.shape[1] // n_head
    n_kv_head = n_kv_head or n_head
    group = n_head // n_kv_head
    out = np.zeros_like(q)
    for h in range(n_head):
        g = h // group
        qh = q[:, h * D:(h + 1) * D]
        kh, vh = k[:, g * D:(g + 1) * D], v[:, g * D:(g + 1) * D]
        for t in range(T):
            p = past + t
            lo = 0 if window is None else max(0, p - window + 1)
            s = (kh[lo:p + 1] @ qh[t]) * scale
            w = softmax_rows(s[None, :])[0]
            out[t, h * D:(h + 1) * D] = w @ vh[lo:p + 1]
    return out


def attention_block(a, W, layer, n_head, scale):
    """Fused projection, split in thirds q|k|v (Gpt2Model.java:81-82), attention, output
    projection with bias (CausalSelfAttention.java:385-408)."""
    p = f"h.{layer}.attn."
    qkv = conv1d(a, W[p + "c_attn.weight"], W[p + "c_attn.bias"])
    E = a.shape[1]
    q, k, v = qkv[:, :E], qkv[:, E:2 * E], qkv[:, 2 * E:]
    o = causal_attention(q, k, v, n_head, scale)
    return conv1d(o, W[p + "c_proj.weight"], W[p + "c_proj.bias"])


def mlp_block(m, W, layer, activation):
    """fc + bias, activation, proj + bias (core/.../generator/MLPBlock.java:250-321)."""
    p = f"h.{layer}.mlp."
    h = conv1d(m, W[p + "c_fc.weight"], W[p + "c_fc.bias"])
    h = ACTIVATIONS[activation](h)
    return conv1d(h, W[p + "c_proj.weight"], W[p + "c_proj.bias"])


def block(x, W, layer, cfg):
    """x1 = x + Attn(LN1(x)); x2 = x1 + MLP(LN2(x1))
    (core/.../generator/TransformerBlock.java:35-41,169-198)."""
    eps = cfg.get("layer_norm_epsilon", 1e-5)
    E, H = cfg["n_embd"], cfg["n_head"]
    scale = 1.0 / math.sqrt(E // H)        # CausalSelfAttention.java:203
    if cfg.get("scale_attn_by_inverse_layer_idx", False):
        scale /= (layer + 1)
    p = f"h.{layer}."
    a = layer_norm(x, W[p + "ln_1.weight"], W[p + "ln_1.bias"], eps)
    x = x + attention_block(a, W, layer, H, scale)
    m = layer_norm(x, W[p + "ln_2.weight"], W[p + "ln_2.bias"], eps)
    return x + mlp_block(m, W, layer, cfg.get("activation_function", "gelu_new"))


def head(x, W, cfg):
    """ln_f, then logits against the token table (tied head: Gpt2Model.java:54-71;
    core/.../model/AbstractGeneratorSampler.java:53-70,112-115)."""
    e = layer_norm(x, W["ln_f.weight"], W["ln_f.bias"], cfg.get("layer_norm_epsilon", 1e-5))
    table = W["wte.weight"] if cfg.get("tie_word_embeddings", True) or "lm_head.weight" not in W \
        else W["lm_head.weight"]
    return e @ table.T


def forward_logits(cfg, W, ids):
    """Logits [T, V] at every position of one whole sequence."""
    T = len(ids)
    x = embed(ids, np.arange(T), W["wte.weight"], W["wpe.weight"])
    for l in range(cfg["n_layer"]):
        x = block(x, W, l, cfg)
    return head(x, W, cfg)


def greedy_generate(cfg, W, prompt, n_new):
    """Arg-max decoding, first maximum wins
    (core/.../model/AbstractGeneratorSampler.java:135-151,161-173)."""
    ids = list(prompt)
    for _ in range(n_new):
        logits = forward_logits(cfg, W, ids)[-1]
        ids.append(int(np.argmax(logits)))
    return ids[len(prompt):]


# --------------------------------------------------------------------------- sampling
class JavaRandom:
    """java.util.Random's 48-bit generator, which the reference seeds per request
    (core/.../model/GenerationEngine.java:89)."""

    def __init__(self, seed):
        self.s = (seed ^ 0x5DEECE66D) & ((1 << 48) - 1)

    def _next(self, bits):
        self.s = (self.s * 0x5DEECE66D + 0xB) & ((1 << 48) - 1)
        return self.s >> (48 - bits)

    def next_float(self):
        return self._next(24) / float(1 << 24)


def top_k_candidate_count(top_k, vocab):
    """AbstractGeneratorSampler.java:256-264."""
    if top_k <= 0:
        raise ValueError("topK must be > 0")
    if top_k < 1.0:
        return max(1, vocab - int(np.float32(top_k) * np.float32(vocab)))
    return min(vocab, int(math.floor(top_k + 0.5)))


def sample_top_k_top_p(logits, temperature, top_k, top_p, uniform_top_p, u):
    """AbstractGeneratorSampler.java:266-323: scale by 1/T, stable sort descending, keep k,
    nucleus until the cumulative probability reaches p (crossing token kept), then walk the
    kept list with pick = u * total."""
    if temperature <= 0:
        raise ValueError("temperature must be > 0 for sampling")
    if top_p is not None and not (0 < top_p <= 1):
        raise ValueError("topP must be in (0, 1]")
    if uniform_top_p is not None and not (0 < uniform_top_p <= 1):
        raise ValueError("uniformTopP must be in (0, 1]")
    if uniform_top_p is not None and top_p is None:
        raise ValueError("uniformTopP requires topP")
    v = np.asarray(logits, dtype=np.float32) / np.float32(temperature)
    V = len(v)
    limit = V if top_k is None else top_k_candidate_count(top_k, V)
    order = np.argsort(-v.astype(np.float64), kind="stable")[:limit]
    mx = float(v.max())
    w = np.exp(v[order].astype(np.float64) - mx)
    total = w.sum()
    if top_p is not None:
        cum = np.cumsum(w / total)
        n = int(np.searchsorted(cum, np.float32(top_p), side="left")) + 1
        n = min(n, len(order))
        order, w = order[:n], w[:n]
        total = w.sum()
        if uniform_top_p is not None:
            return int(order[min(int(np.float32(u) * len(order)), len(order) - 1)])
    pick = u * total
    for idx, wi in zip(order, w):
        pick -= wi
        if pick <= 0:
            return int(idx)
    return int(order[-1])
