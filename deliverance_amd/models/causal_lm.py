"""The model every architecture becomes: embedding, a run order over blocks, final norm, head.

It is assembled from a ``ModelConfig`` and parameters under the parts' local names, and it
knows nothing of any particular architecture.  One forward call runs the tokens of one step:
embed -> each entry of the run order -> norm of the wanted rows -> logits of the wanted rows.
Reference: core/src/main/java/io/teknek/deliverance/model/AbstractModel.java:1097-1118 (layer
loop); the final norm and the head act on sampled rows only
(core/.../model/AbstractGeneratorSampler.java:112-115).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.specs import ModelConfig
from ..kernels import ops
from ..parts import Block, StepContext, build_norm, build_position, to_matrix, to_vector
from ..registry import Architecture, ModelSupport, read_config_json
from ..weights.loader import load_declared


class CausalLM:
    def __init__(self, config: ModelConfig, params: dict, dtype: torch.dtype, device):
        self.config = config
        self.dtype = dtype
        self.device = torch.device(device)
        emb = params["embed"]
        # Tables are read by row in their stored dtype; in the 32-bit path they are widened.
        self.token_table = to_vector(emb["tokens"], dtype, device)
        if tuple(self.token_table.shape) != (config.vocab_size, config.width):
            raise ValueError(f"token table is {list(self.token_table.shape)}, expected "
                             f"{[config.vocab_size, config.width]}")
        self.embed_position = build_position(config.embed_position, emb.get("positions", {}), dtype, device)
        self.blocks: List[Block] = [Block(spec, p, dtype, device)
                                    for spec, p in zip(config.layers, params["layers"])]
        self.final_norm = None if config.final_norm is None else \
            build_norm(config.final_norm, params["final_norm"], dtype, device)
        head = params["head"]["weight"]
        if head is emb["tokens"] and self.token_table.dtype == dtype:
            self.head_weight = self.token_table            # tied: one buffer, two uses
        else:
            self.head_weight = to_matrix(head, dtype, device)
        for call in config.schedule:
            if not (0 <= call.layer < len(self.blocks)):
                raise ValueError(f"run order names layer {call.layer}, the model has {len(self.blocks)}")

    @property
    def graph_safe(self) -> bool:
        """Whether every part allows a decode step to be replayed from a recorded HIP graph."""
        return all(b.mixer.graph_safe and (b.feed_forward is None or b.feed_forward.graph_safe) for b in self.blocks)

    # ---- what the cache must provide -----------------------------------------------------
    def cache_needs(self) -> Dict[int, object]:
        """cache slot -> KVNeed / StateNeed of the layer call that writes it."""
        needs: Dict[int, object] = {}
        for call in self.config.schedule:
            need = self.blocks[call.layer].mixer.cache_need()
            if need is None:
                continue
            if call.write:
                if call.cache in needs:
                    raise ValueError(f"cache slot {call.cache} is written by two layer calls")
                needs[call.cache] = need
        for call in self.config.schedule:
            need = self.blocks[call.layer].mixer.cache_need()
            if need is not None and not call.write:
                if call.cache not in needs:
                    raise ValueError(f"layer {call.layer} reads cache slot {call.cache} that nothing writes")
                if needs[call.cache] != need:
                    raise ValueError(f"layer {call.layer} reads cache slot {call.cache} of another shape")
        return needs

    # ---- one step ----------------------------------------------------------------------------
    def forward(self, ctx: StepContext, want_rows: Optional[torch.Tensor], n_want: int) -> torch.Tensor:
        """Logits [n_want, V] (32-bit) of rows ``want_rows`` (int32, device) of this step."""
        with ops.pinned_stream():
            return self._forward(ctx, want_rows, n_want)

    def _forward(self, ctx: StepContext, want_rows: Optional[torch.Tensor], n_want: int) -> torch.Tensor:
        N = ctx.n_tokens
        x = ctx.buf("residual", N, self.config.width, torch.float32)
        ops.embed(ctx.tokens, ctx.positions, self.token_table, self.embed_position.embed_table(), x,
                  self.config.embed_scale)
        debug = ctx.debug_hook is not None          # the reference's stages: AbstractModel.java:1100,1107
        if debug:
            ctx.emit(-1, "input", x)
        for call in self.config.schedule:
            self.blocks[call.layer].forward(ctx, x, call)
            if debug:
                ctx.emit(call.layer, "layer_output", x)
        logits = ctx.buf("logits", n_want, self.config.vocab_size, torch.float32)
        if n_want == 0:
            return logits
        ln = None if self.final_norm is None else self.final_norm.fusable_params()
        if ln is not None and ops.can_fuse_ln(n_want, x, self.head_weight):
            gain, bias, eps = ln                   # few wanted rows: norm and head in one kernel
            ops.linear_ln(x, want_rows, n_want, gain, bias, eps, self.head_weight, None, logits)
        else:
            if self.final_norm is not None:
                e = self.final_norm.forward(ctx, x, rows=want_rows, n_rows=n_want, out_name="final_norm")
            else:
                e = ops.copy_rows(x, ctx.buf("final_norm", n_want, self.config.width, ctx.dtype), rows=want_rows)
            ops.linear(e, self.head_weight, None, logits)
        if self.config.logit_multiplier != 1.0:     # (an architecture's constant; GPT-2 has none)
            ops.copy_rows(logits, logits, scale=1.0 / self.config.logit_multiplier)
        return logits


def load_model(folder: str, dtype: torch.dtype, device) -> CausalLM:
    """config.json picks the architecture; its tensors are read by name and bound to parts."""
    cfg_dict = read_config_json(folder)
    arch: Architecture = ModelSupport.detect(cfg_dict)
    mc = arch.read_config(cfg_dict)
    tensors = load_declared(folder, arch.declare_tensors(mc), ignore=arch.ignore_tensors,
                            strip_prefixes=arch.strip_prefixes)
    return CausalLM(mc, arch.bind_tensors(mc, tensors), dtype, device)
