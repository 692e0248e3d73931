"""The arrangement of one block: optional norms around a mixer and a feed-forward, each
adding into the 32-bit residual stream.
Reference: core/src/main/java/io/teknek/deliverance/generator/TransformerBlock.java:161-200
(five optional norm places :26-32; GPT-2 uses the two pre-norms :35-41)."""
from __future__ import annotations

import torch

from .base import StepContext, build_feed_forward, build_mixer, build_norm


class Block:
    def __init__(self, spec, params, dtype, device):
        def norm(s, key):
            return None if s is None else build_norm(s, params[key], dtype, device)

        self.pre_mixer_norm = norm(spec.pre_mixer_norm, "pre_mixer_norm")
        self.post_mixer_norm = norm(spec.post_mixer_norm, "post_mixer_norm")
        self.pre_ff_norm = norm(spec.pre_ff_norm, "pre_ff_norm")
        self.post_ff_norm = norm(spec.post_ff_norm, "post_ff_norm")
        self.mixer = build_mixer(spec.mixer, params["mixer"], dtype, device)
        self.feed_forward = None if spec.feed_forward is None else \
            build_feed_forward(spec.feed_forward, params["feed_forward"], dtype, device)
        if self.post_mixer_norm is not None or self.post_ff_norm is not None:
            # A norm after a part acts on the part's output before the residual add, which
            # needs the part to write to a buffer of its own instead of into the stream.
            raise NotImplementedError("post-part norms are not wired yet")

    @staticmethod
    def _normed(ctx, x, pre):
        if pre is not None:
            return pre.forward(ctx, x)
        h = ctx.buf("norm", x.shape[0], x.shape[1], ctx.dtype)
        h.copy_(x)
        return h

    def forward(self, ctx: StepContext, x: torch.Tensor, call) -> None:
        # A part may offer `forward_normed(ctx, norm, x, ...)`: it then applies the norm itself
        # (fused into its first product) and returns True, or returns False to decline this step.
        fused = getattr(self.mixer, "forward_normed", None)
        if not (fused is not None and self.pre_mixer_norm is not None and fused(ctx, self.pre_mixer_norm, x, call)):
            self.mixer.forward(ctx, self._normed(ctx, x, self.pre_mixer_norm), x, call)
        if self.feed_forward is not None:
            fused = getattr(self.feed_forward, "forward_normed", None)
            if not (fused is not None and self.pre_ff_norm is not None and fused(ctx, self.pre_ff_norm, x)):
                self.feed_forward.forward(ctx, self._normed(ctx, x, self.pre_ff_norm), x)
