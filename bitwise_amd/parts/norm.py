"""RMSNorm: y = (x * 1/sqrt(mean(x^2) + eps)) * weight (src/kernels.cpp:264-271)."""

from __future__ import annotations

from typing import Dict

import torch

from ..csrc import ops
from .base import Norm, TensorSpec, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """params: width, eps.  tensor: weight [width].  The sum of squares, the root and both
    products are 32-bit; the output has the mode's activation dtype."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width = int(params["width"])
        self.eps = float(params["eps"])
        self.weight = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.width,), "norm")}

    def bind(self, tensors) -> None:
        self.weight = tensors["weight"].to(self.rt.device).contiguous()

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def forward(self, ctx, x: torch.Tensor, out_name: str = "normed", rows: int | None = None) -> torch.Tensor:
        rows = ctx.rows if rows is None else rows
        out = ctx.ws.buffer(out_name, self.width, self.rt.act_dtype)
        ops.rmsnorm(x, self.weight, out, rows, self.eps)
        return out
