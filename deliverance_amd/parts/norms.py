"""LayerNorm as a part.  Formula: core/src/main/java/io/teknek/deliverance/generator/
LayerNorm.java:127-150 (mean, biased variance, eps inside the root, gain and bias)."""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Norm, StepContext, register_norm, to_vector


class LayerNorm(Norm):
    def __init__(self, spec, params, dtype, device):
        self.width = spec.width
        self.eps = float(spec.eps)
        self.weight = to_vector(params["weight"], dtype, device)
        self.bias = to_vector(params.get("bias"), dtype, device) if spec.bias else None
        if self.weight.numel() != self.width:
            raise ValueError(f"LayerNorm gain has {self.weight.numel()} entries for width {self.width}")

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                n_rows: Optional[int] = None, out_name: str = "norm",
                out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        R = x.shape[0] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.buf(out_name, R, self.width, out_dtype or ctx.dtype)
        return ops.layernorm(x, self.weight, self.bias, self.eps, out, rows)

    def fusable_params(self):
        return self.weight, self.bias, self.eps


register_norm("layernorm", LayerNorm)
