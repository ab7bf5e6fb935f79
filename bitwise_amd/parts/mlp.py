"""Dense SwiGLU feed-forward (src/model.cpp:301-305, src/kernels.cpp:291-298):
one stacked product [gate; up], h = g * (1/(1+exp(-g))) * u, down projection added into the
residual stream."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import FeedForward, TensorSpec, register_feed_forward
from .linear import Linear


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """params: width, inter.  tensors: gate_proj/up_proj/down_proj .weight."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.width, self.inter = int(params["width"]), int(params["inter"])
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {
            "gate_proj.weight": TensorSpec((self.inter, self.width)),
            "up_proj.weight": TensorSpec((self.inter, self.width)),
            "down_proj.weight": TensorSpec((self.width, self.inter)),
        }

    def bind(self, tensors) -> None:
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        if g.dtype != u.dtype:
            raise ValueError("gate and up projections must be stored in one dtype to be stacked")
        self.gate_up = Linear(torch.cat([g, u], dim=0), self.rt)
        self.down = Linear(tensors["down_proj.weight"], self.rt)

    def weight_bytes(self) -> int:
        return self.gate_up.nbytes() + self.down.nbytes()

    def forward_with_norm(self, ctx, x, norm, residual) -> bool:
        """Decode steps of few rows: norm, the stacked product and SwiGLU are one kernel."""
        from .norm import RMSNorm
        rt, ws = self.rt, ctx.ws
        if not (rt.bf16 and isinstance(norm, RMSNorm) and self.gate_up.mfma and self.down.mfma
                and ops.can_fuse_norm(ctx.rows, self.gate_up.weight, x, columns=32, stacked=2)):
            return False
        act = ws.buffer("mlp_h", self.inter, torch.bfloat16)
        ops.norm_gemm_bf16(x, norm.weight, norm.eps, self.gate_up.weight, act, ctx.rows, ops.EPI_SWIGLU_BF16)
        self.down.add_into(ws, act, residual, ctx.rows)
        return True

    def forward(self, ctx, h, residual) -> None:
        rt, ws, rows = self.rt, ctx.ws, ctx.rows
        if self.gate_up.mfma:
            act = ws.buffer("mlp_h", self.inter, torch.bfloat16)
            ops.gemm_bf16(h, self.gate_up.weight, act, rows, ops.EPI_SWIGLU_BF16)   # SwiGLU in the epilogue
        else:
            gu = ws.buffer("gate_up", 2 * self.inter, torch.float32)
            self.gate_up.store(ws, h, gu, rows)
            act32 = ws.buffer("mlp_h32", self.inter, torch.float32)
            ops.swiglu_f32(gu, act32, rows)
            if rt.bf16:
                # bfloat16 mode rounds the activation here whatever dtype the weights are stored in, so that
                # the mode has one set of rounding points (a 32-bit down projection widens it again)
                act = ws.buffer("mlp_h", self.inter, torch.bfloat16)
                ops.convert(act32, act, rows)
            else:
                act = act32
        self.down.add_into(ws, act, residual, rows)
