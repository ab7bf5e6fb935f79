"""Token embedding and the language-model head (src/model.cpp:274, :308-321)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import Embedding, Head, TensorSpec, register_embedding, register_head
from .linear import Linear


@register_embedding("embedding")
class TokenEmbedding(Embedding):
    """params: vocab, width.  tensor: weight [vocab, width], gathered as 32-bit rows."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.vocab, self.width = int(params["vocab"]), int(params["width"])
        self.weight: Optional[torch.Tensor] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.vocab, self.width), "embedding")}

    def bind(self, tensors) -> None:
        self.weight = tensors["weight"].to(self.rt.device).contiguous()

    def weight_bytes(self) -> int:
        return 0      # a step reads one row per token, not the table

    def forward(self, ctx) -> torch.Tensor:
        x = ctx.ws.buffer("residual", self.width, torch.float32)
        # (a step launched ahead of its tokens names them by the step before: ``ctx.token_feedback``)
        ops.embed(ctx.tokens[:ctx.rows], self.weight, x, getattr(ctx, "token_feedback", None))
        return x


@register_head("lm_head")
class LMHead(Head):
    """params: vocab, width, tied.  tensor: weight [vocab, width] unless tied to the embedding
    (src/model.cpp:170-171).  Only the wanted rows are normed and projected."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.vocab, self.width, self.tied = int(params["vocab"]), int(params["width"]), bool(params["tied"])
        self.linear: Optional[Linear] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {} if self.tied else {"weight": TensorSpec((self.vocab, self.width), "linear")}

    def bind(self, tensors, embedding=None) -> None:
        if self.tied:
            table = getattr(embedding, "weight", None)
            if table is None or tuple(table.shape) != (self.vocab, self.width):
                raise ValueError("a tied head needs an embedding part with a table [vocab, width]")
            self.linear = Linear(table, self.rt)     # the same device tensor, not a copy
        else:
            self.linear = Linear(tensors["weight"], self.rt)

    def weight_bytes(self) -> int:
        return self.linear.nbytes()

    def forward(self, ctx, x: torch.Tensor, norm, count: int) -> torch.Tensor:
        """Final norm and projection of ``count`` rows; few rows: both are one kernel (the same bits)."""
        from .norm import RMSNorm
        ws = ctx.ws
        logits = ws.buffer("logits", self.vocab, torch.float32, rows=ws.max_logit_rows)
        if (self.rt.bf16 and isinstance(norm, RMSNorm) and self.linear.mfma
                and ops.can_fuse_norm(count, self.linear.weight, x)):
            ops.norm_gemm_bf16(x, norm.weight, norm.eps, self.linear.weight, logits, count, ops.EPI_F32)
            return logits
        normed = norm.forward(ctx, x, out_name="final_normed", rows=count)
        self.linear.store(ws, normed, logits, count)
        return logits
