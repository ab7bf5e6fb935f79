"""Rotary position encoding in the rotate-half layout (src/kernels.cpp:273-289).

inv_freq[i] = 1.0f / powf(theta, float(2i)/float(hd)) (src/model.cpp:220-225) and
angle = float(pos) * inv_freq[i] are 32-bit values, as in the reference; cosine and sine of
that 32-bit angle are evaluated in double and rounded once.  The tables are built on the host
for all positions up to ``max_positions`` and read by the kernels.
"""

from __future__ import annotations

import numpy as np
import torch

from .base import PositionEncoding, register_position_encoding


@register_position_encoding("rope")
class RotaryTable(PositionEncoding):
    """params: theta, head_dim, max_positions.  No checkpoint tensors."""

    graph_safe = True
    launches_through_ops = True

    def __init__(self, params, runtime):
        super().__init__(params, runtime)
        self.theta = float(params["theta"])
        self.head_dim = int(params["head_dim"])
        self.max_positions = int(params["max_positions"])
        if self.head_dim % 2:
            raise ValueError("rotary encoding needs an even head size")
        self.rotary_dim = self.head_dim          # whole heads are rotated
        self._cos = self._sin = None

    def _build(self) -> None:
        runtime = self.rt
        half = self.head_dim // 2
        i = np.arange(half, dtype=np.float32)
        expo = (np.float32(2.0) * i) / np.float32(self.head_dim)
        inv_freq = (np.float32(1.0) / np.power(np.float32(self.theta), expo, dtype=np.float32)).astype(np.float32)
        pos = np.arange(self.max_positions, dtype=np.float32)[:, None]
        angle = (pos * inv_freq[None, :]).astype(np.float32).astype(np.float64)
        self._cos = torch.from_numpy(np.cos(angle).astype(np.float32)).to(runtime.device).contiguous()
        self._sin = torch.from_numpy(np.sin(angle).astype(np.float32)).to(runtime.device).contiguous()

    def tables(self):
        if self._cos is None:
            self._build()
        return self._cos, self._sin

    @classmethod
    def shared(cls, params, runtime) -> "RotaryTable":
        key = ("rope", float(params["theta"]), int(params["head_dim"]), int(params["max_positions"]))
        return runtime.shared(key, lambda: cls(params, runtime))
