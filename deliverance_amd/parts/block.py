"""The arrangement of one block: optional norms around a mixer and a feed-forward, each
adding into the 32-bit residual stream.
Reference: core/src/main/java/io/teknek/deliverance/generator/TransformerBlock.java:161-200
(five optional norm places :26-32; GPT-2 uses the two pre-norms :35-41; a norm after a part acts
on the part's output before the residual add :172-176,184-188; the part's output may join the stream
times a constant :260-272; the fifth norm acts on the stream at the block's end :199)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import StepContext, build_feed_forward, build_mixer, build_norm


class Block:
    def __init__(self, spec, params, dtype, device):
        def norm(s, key):
            return None if s is None else build_norm(s, params[key], dtype, device)

        self.pre_mixer_norm = norm(spec.pre_mixer_norm, "pre_mixer_norm")
        self.post_mixer_norm = norm(spec.post_mixer_norm, "post_mixer_norm")
        self.pre_ff_norm = norm(spec.pre_ff_norm, "pre_ff_norm")
        self.post_ff_norm = norm(spec.post_ff_norm, "post_ff_norm")
        self.post_block_norm = norm(getattr(spec, "post_block_norm", None), "post_block_norm")
        self.residual_multiplier = float(getattr(spec, "residual_multiplier", 1.0))
        self.mixer = build_mixer(spec.mixer, params["mixer"], dtype, device)
        self.feed_forward = None if spec.feed_forward is None else \
            build_feed_forward(spec.feed_forward, params["feed_forward"], dtype, device)

    @staticmethod
    def _normed(ctx, x, pre):
        if pre is not None:
            return pre.forward(ctx, x)
        h = ctx.buf("norm", x.shape[0], x.shape[1], ctx.dtype)      # no norm in front: the stream, converted
        return ops.copy_rows(x, h)

    def _part(self, ctx, x, pre, post, run, run_normed):
        """One part of the block.  Parts add into the tensor they are given.  Without a norm behind
        the part (and without a multiplier) that tensor is the residual stream; else the part adds
        into a buffer of its own (cleared by a fill kernel of the engine's, so that a recorded step
        holds no memset), whose norm, kept in 32-bit, times the multiplier is then added to the stream."""
        target = x
        own = post is not None or self.residual_multiplier != 1.0
        if own:
            target = ops.fill_zero(ctx.buf("part_out", x.shape[0], x.shape[1], torch.float32))
        # A part may offer `forward_normed(ctx, norm, x, ...)`: it then applies the norm in front
        # of it itself (fused into its first product) and returns True, or returns False to
        # decline this step.  That needs the part's input and the tensor it adds into to be the same.
        if not (not own and pre is not None and run_normed is not None and run_normed(pre)):
            run(Block._normed(ctx, x, pre), target)
        if own:
            out = target if post is None else post.forward(ctx, target, out_name="post_norm", out_dtype=torch.float32)
            ops.copy_rows(out, x, accumulate=True, scale=self.residual_multiplier)

    def forward(self, ctx: StepContext, x: torch.Tensor, call) -> None:
        fused = getattr(self.mixer, "forward_normed", None)
        self._part(ctx, x, self.pre_mixer_norm, self.post_mixer_norm,
                   lambda h, into: self.mixer.forward(ctx, h, into, call),
                   None if fused is None else (lambda norm: fused(ctx, norm, x, call)))
        if ctx.debug_hook is not None:
            ctx.emit(call.layer, "post_attention_residual", x)
        if self.feed_forward is not None:
            fused = getattr(self.feed_forward, "forward_normed", None)
            self._part(ctx, x, self.pre_ff_norm, self.post_ff_norm,
                       lambda h, into: self.feed_forward.forward(ctx, h, into),
                       None if fused is None else (lambda norm: fused(ctx, norm, x)))
            if ctx.debug_hook is not None:
                ctx.emit(call.layer, "post_ff_residual", x)
        if self.post_block_norm is not None:                # the stream itself, normalised in place
            ops.copy_rows(self.post_block_norm.forward(ctx, x, out_name="post_norm", out_dtype=torch.float32), x)
