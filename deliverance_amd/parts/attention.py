"""Causal self-attention over the paged cache, as a mixer.

Fused projection to q | k | v (+ bias), optional position encoding of q and k, write of the
new k and v rows into the cache slot, attention of every row over its sequence's pages, and
the output projection (+ bias) added into the residual stream.
Reference: core/src/main/java/io/teknek/deliverance/generator/CausalSelfAttention.java:226-420
(projections :266-291, cache write :315-336, scores/softmax/weighted sum :458-532, output
projection :385-408); the residual add is TransformerBlock.java:176.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import (KVNeed, Mixer, StepContext, build_position, register_mixer, to_matrix, to_vector)


class CausalSelfAttention(Mixer):
    graph_safe = True

    def __init__(self, spec, params, dtype, device):
        self.spec = spec
        self.n_heads, self.n_kv_heads, self.head_dim = spec.n_heads, spec.n_kv_heads, spec.head_dim
        if self.n_heads % self.n_kv_heads != 0:
            raise ValueError(f"{self.n_heads} query heads are not a multiple of {self.n_kv_heads} key heads")
        # Any head size up to 256 runs: multiples of 16 on the matrix-core attention kernels in bfloat16,
        # the others (and everything in 32-bit) on the plain attention kernel.
        if not (1 <= self.head_dim <= ops.MAX_HEAD_DIM):
            raise ValueError(f"head size {self.head_dim} is outside 1..{ops.MAX_HEAD_DIM}")
        self.q_cols = self.n_heads * self.head_dim
        self.kv_cols = self.n_kv_heads * self.head_dim
        self.qkv_cols = self.q_cols + 2 * self.kv_cols
        self.scale = float(spec.scale)
        self.window = spec.window
        self.qkv_weight = to_matrix(params["qkv_weight"], dtype, device)
        self.out_weight = to_matrix(params["out_weight"], dtype, device)
        self.qkv_bias = to_vector(params.get("qkv_bias"), dtype, device) if spec.qkv_bias else None
        self.out_bias = to_vector(params.get("out_bias"), dtype, device) if spec.out_bias else None
        if tuple(self.qkv_weight.shape) != (self.qkv_cols, spec.width):
            raise ValueError(f"qkv weight is {list(self.qkv_weight.shape)}, expected {[self.qkv_cols, spec.width]}")
        if tuple(self.out_weight.shape) != (spec.width, self.q_cols):
            raise ValueError(f"output weight is {list(self.out_weight.shape)}, expected {[spec.width, self.q_cols]}")
        self.position = None
        if spec.position is not None and spec.position.kind != "none":
            self.position = build_position(spec.position, params.get("position", {}), dtype, device)

    def cache_need(self):
        return KVNeed(self.n_kv_heads, self.head_dim, self.window)

    def forward_normed(self, ctx: StepContext, norm, x: torch.Tensor, call) -> bool:
        """Small steps: LayerNorm, the q|k|v projection and the cache write in one kernel."""
        N = x.shape[0]
        ln = norm.fusable_params()
        if ln is None or self.position is not None or not ops.can_fuse_ln(N, x, self.qkv_weight):
            return False
        gain, bias, eps = ln
        qkv = ctx.buf("qkv", N, self.qkv_cols, ctx.dtype)
        slot = ctx.cache.kv[call.cache]
        group = ctx.group_of(call.cache)
        ops.linear_ln(x, None, N, gain, bias, eps, self.qkv_weight, self.qkv_bias, qkv,
                      kv_cache=slot if call.write else None, slot_map=ctx.slot_maps[group] if call.write else None,
                      q_cols=self.q_cols)
        self._attend(ctx, qkv, x, slot, group, call)
        return True

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor, call) -> None:
        N = h.shape[0]
        qkv = ctx.buf("qkv", N, self.qkv_cols, ctx.dtype)
        slot = ctx.cache.kv[call.cache]
        group = ctx.group_of(call.cache)
        if self.position is None and call.write:
            # the new keys and values go to the cache in the projection's epilogue
            ops.linear(h, self.qkv_weight, self.qkv_bias, qkv, kv_cache=slot, slot_map=ctx.slot_maps[group],
                       q_cols=self.q_cols)
        else:
            ops.linear(h, self.qkv_weight, self.qkv_bias, qkv)
            if self.position is not None:
                self.position.apply_qk(ctx, qkv, self.n_heads, self.n_kv_heads, self.head_dim)
            if call.write:
                ops.kv_write(qkv, self.q_cols, self.q_cols + self.kv_cols, slot, ctx.slot_maps[group],
                             self.n_kv_heads, self.head_dim)
        self._attend(ctx, qkv, x, slot, group, call)

    def _attend(self, ctx: StepContext, qkv: torch.Tensor, x: torch.Tensor, slot: torch.Tensor, group: int,
                call) -> None:
        N = qkv.shape[0]
        o = ctx.buf("attn_out", N, self.q_cols, ctx.dtype)
        ops.paged_attention(ctx, qkv[:, :self.q_cols], slot, group, self.n_heads, self.scale, self.window, o)
        if ctx.debug_hook is not None:      # the reference's stage names (CausalSelfAttention.java:299-301,384)
            ctx.emit(call.layer, "query_projection", qkv[:, :self.q_cols])
            ctx.emit(call.layer, "key_projection", qkv[:, self.q_cols:self.q_cols + self.kv_cols])
            ctx.emit(call.layer, "value_projection", qkv[:, self.q_cols + self.kv_cols:])
            ctx.emit(call.layer, "attention_value", o)
            # the output projection before its bias (CausalSelfAttention.java:406), worked out once more for the hook
            ctx.emit(call.layer, "attention_output",
                     ops.linear(o, self.out_weight, None, ctx.buf("attn_proj_debug", N, x.shape[1], torch.float32)))
        ops.linear(o, self.out_weight, self.out_bias, x, accumulate=True)


register_mixer("attention", CausalSelfAttention)
