"""A weight matrix [out, in] and the matrix product that fits its dtype and the mode.

Reference: y[m][n] = sum_k x[m][k] * W[n][k], W as stored by the checkpoint, no bias
(src/kernels.cpp:236-244).  bfloat16 weights run on the matrix cores in bfloat16 mode; a
weight stored in 32-bit stays 32-bit and runs through the 32-bit kernel in either mode.

The reference's architecture has no biases.  A part of another architecture that has one passes ``bias``:
y = (the product's sum) + bias[n], one 32-bit addition behind the sum, by a kernel of its own (the fused
epilogues of the products stay what they are), and where the product is added into the residual stream the
biased product is formed first and added whole.
"""

from __future__ import annotations

import torch

from ..csrc import ops


class Linear:
    def __init__(self, weight: torch.Tensor, runtime, bias: torch.Tensor | None = None):
        if weight.dim() != 2 or weight.dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("a linear weight must be a bfloat16 or float32 matrix")
        self.rt = runtime
        self.weight = weight.to(runtime.device).contiguous()
        self.bias = None
        if bias is not None:
            if bias.dim() != 1 or bias.shape[0] != weight.shape[0]:
                raise ValueError(f"a bias of {tuple(bias.shape)} does not fit a weight of {tuple(weight.shape)}")
            self.bias = bias.to(runtime.device).float().contiguous()      # (widening is exact)
        self.out_features, self.in_features = self.weight.shape
        self.mfma = runtime.bf16 and self.weight.dtype == torch.bfloat16
        if self.mfma and self.in_features % 8:
            raise ValueError(f"bfloat16 matrix product: inner size {self.in_features} must be a multiple of 8")

    def nbytes(self) -> int:
        return self.weight.numel() * self.weight.element_size() + (0 if self.bias is None else self.bias.numel() * 4)

    def _x32(self, ws, x: torch.Tensor, rows: int) -> torch.Tensor:
        if x.dtype == torch.float32:
            return x
        buf = ws.buffer("linear_x32", x.shape[1], torch.float32)
        ops.convert(x, buf, rows)
        return buf

    def store(self, ws, x: torch.Tensor, out: torch.Tensor, rows: int) -> None:
        """out[:rows] = x[:rows] @ W.T (out float32, or bfloat16 on the matrix-core path).  ``ws`` is the
        step's workspace (temporaries for a weight whose dtype is not the mode's)."""
        if self.bias is not None:
            # the 32-bit sums, the bias, then the rounding if the caller wants bfloat16
            y = out if out.dtype == torch.float32 else ws.buffer("linear_y32", self.out_features, torch.float32)
            if self.mfma:
                ops.gemm_bf16(x, self.weight, y, rows, ops.EPI_F32)
            else:
                ops.gemm_f32(self._x32(ws, x, rows), self.weight, y, rows)
            ops.add_bias(y, self.bias, rows)
            if y is not out:
                ops.convert(y, out, rows)
        elif self.mfma:
            ops.gemm_bf16(x, self.weight, out, rows, ops.EPI_BF16 if out.dtype == torch.bfloat16 else ops.EPI_F32)
        elif out.dtype == torch.float32:
            ops.gemm_f32(self._x32(ws, x, rows), self.weight, out, rows)
        else:
            tmp = ws.buffer("linear_y32", self.out_features, torch.float32)
            ops.gemm_f32(self._x32(ws, x, rows), self.weight, tmp, rows)
            ops.convert(tmp, out, rows)

    def add_into(self, ws, x: torch.Tensor, residual: torch.Tensor, rows: int) -> None:
        """residual[:rows] += x[:rows] @ W.T, the sum in 32-bit (src/model.cpp:300, :305)."""
        if self.bias is not None:
            y = ws.buffer("linear_biased", self.out_features, torch.float32)
            self.store(ws, x, y, rows)
            ops.add_(residual, y, rows)
            return
        if self.mfma:
            # 17 rows or more and a long inner size: every 2048-segment of it gets workgroups of its own, which meet
            # in device scratch.  For up to 64 rows (or a few blocks of 64) that is a fixed size; for a prompt portion
            # it holds the segments' sums whole and is sized for the longest step, so that one buffer serves every
            # portion.
            scratch = None
            floats, counters = ops.gemm_add_scratch(rows, self.out_features, self.in_features) if rows > 16 else (0, 0)
            if floats and rows > 64:
                longest = ops.gemm_add_scratch(ws.max_rows, self.out_features, self.in_features)
                floats, counters = max(floats, longest[0]), max(counters, longest[1])
            if floats:
                scratch = (ws.buffer("gemm_add_split", floats, torch.float32, rows=1),
                           ws.buffer("gemm_add_split_count", counters, torch.int32, rows=1))
            ops.gemm_bf16(x, self.weight, residual, rows, ops.EPI_ADD_F32, scratch=scratch)
        else:
            ops.gemm_f32(self._x32(ws, x, rows), self.weight, residual, rows, accumulate=True)
