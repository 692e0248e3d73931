"""Dense feed-forward: fc (+ bias), activation, proj (+ bias), added into the residual stream.
Reference: core/src/main/java/io/teknek/deliverance/generator/MLPBlock.java:250-321 (the
two-bias, no-gate form GPT-2 uses, :93-114); residual add TransformerBlock.java:188."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FeedForward, StepContext, register_feed_forward, to_matrix, to_vector


class DenseFeedForward(FeedForward):
    graph_safe = True

    def __init__(self, spec, params, dtype, device):
        self.width, self.inner, self.activation = spec.width, spec.inner, spec.activation
        if self.activation not in ops.ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}")
        self.fc_weight = to_matrix(params["fc_weight"], dtype, device)
        self.proj_weight = to_matrix(params["proj_weight"], dtype, device)
        self.fc_bias = to_vector(params.get("fc_bias"), dtype, device) if spec.bias else None
        self.proj_bias = to_vector(params.get("proj_bias"), dtype, device) if spec.bias else None
        if tuple(self.fc_weight.shape) != (self.inner, self.width):
            raise ValueError(f"fc weight is {list(self.fc_weight.shape)}, expected {[self.inner, self.width]}")
        if tuple(self.proj_weight.shape) != (self.width, self.inner):
            raise ValueError(f"proj weight is {list(self.proj_weight.shape)}, expected {[self.width, self.inner]}")

    def forward_normed(self, ctx: StepContext, norm, x: torch.Tensor) -> bool:
        """Small steps: LayerNorm, fc, bias and activation in one kernel."""
        N = x.shape[0]
        ln = norm.fusable_params()
        if ln is None or not ops.can_fuse_ln(N, x, self.fc_weight):
            return False
        gain, bias, eps = ln
        mid = ctx.buf("ff_mid", N, self.inner, ctx.dtype)
        ops.linear_ln(x, None, N, gain, bias, eps, self.fc_weight, self.fc_bias, mid, act=self.activation)
        ops.linear(mid, self.proj_weight, self.proj_bias, x, accumulate=True)
        return True

    def forward(self, ctx: StepContext, h: torch.Tensor, x: torch.Tensor) -> None:
        N = h.shape[0]
        mid = ctx.buf("ff_mid", N, self.inner, ctx.dtype)
        ops.linear(h, self.fc_weight, self.fc_bias, mid, act=self.activation)
        ops.linear(mid, self.proj_weight, self.proj_bias, x, accumulate=True)


register_feed_forward("dense", DenseFeedForward)
