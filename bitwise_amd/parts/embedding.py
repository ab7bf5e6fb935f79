"""Token embedding and the language-model head (src/model.cpp:274, :308-321)."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..csrc import ops
from .base import Part, TensorSpec
from .linear import Linear


class Embedding(Part):
    """params: vocab, width.  tensor: weight [vocab, width], gathered as 32-bit rows."""

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
        x = self.rt.buffer("residual", self.width, torch.float32)
        ops.embed(ctx.tokens[:ctx.rows], self.weight, x)
        return x


class LMHead(Part):
    """params: vocab, width, tied.  tensor: weight [vocab, width] unless tied to the embedding
    (src/model.cpp:170-171).  Only the wanted rows are normed and projected."""

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.vocab, self.width, self.tied = int(params["vocab"]), int(params["width"]), bool(params["tied"])
        self.linear: Optional[Linear] = None

    def tensors(self) -> Dict[str, TensorSpec]:
        return {} if self.tied else {"weight": TensorSpec((self.vocab, self.width), "linear")}

    def bind(self, tensors, embedding: Optional[Embedding] = None) -> None:
        if self.tied:
            self.linear = Linear(embedding.weight, self.rt)     # the same device tensor, not a copy
        else:
            self.linear = Linear(tensors["weight"], self.rt)

    def weight_bytes(self) -> int:
        return self.linear.nbytes()

    def forward_with_norm(self, ctx, x: torch.Tensor, norm, count: int):
        """Few wanted rows: the final norm and the head product are one kernel.  Returns the
        logits buffer, or None if this step cannot be fused."""
        from .norm import RMSNorm
        if not (self.rt.bf16 and isinstance(norm, RMSNorm) and self.linear.mfma
                and ops.can_fuse_norm(count, self.linear.weight, x)):
            return None
        logits = self.rt.buffer("logits", self.vocab, torch.float32, rows=self.rt.max_logit_rows)
        ops.norm_gemm_bf16(x, norm.weight, norm.eps, self.linear.weight, logits, count, ops.EPI_F32)
        return logits

    def forward(self, ctx, normed: torch.Tensor, count: int) -> torch.Tensor:
        logits = self.rt.buffer("logits", self.vocab, torch.float32, rows=self.rt.max_logit_rows)
        self.linear.store(normed, logits, count)
        return logits
