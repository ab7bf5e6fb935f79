"""What every part shares on the device: precision mode, scratch buffers, position tables."""

from __future__ import annotations

from typing import Any, Callable, Dict, Tuple

import torch

MODES = ("bfloat16", "float32")


class Runtime:
    """Device, precision mode and persistent scratch memory of one model instance.

    mode "bfloat16": the kernels and precisions of serving (bfloat16 operands on the matrix
    cores, 32-bit accumulation, 32-bit residual stream, bfloat16 cache).  mode "float32":
    everything in true 32-bit with plain fused multiply-adds.  Scratch buffers are made once
    for ``max_rows`` rows and never move, so captured HIP graphs stay valid.
    """

    def __init__(self, mode: str = "bfloat16", device: str | torch.device | None = "cuda:0", max_rows: int = 256,
                 page_size: int = 16, max_logit_rows: int | None = None):
        if mode not in MODES:
            raise ValueError(f"dtype must be one of {MODES}, got {mode!r}")
        self.mode = mode
        # device None: the model is only described (tensor names and shapes), nothing can run
        self.device = None if device is None else torch.device(device)
        if self.device is not None and self.device.type != "cuda":
            raise RuntimeError("bitwise_amd runs on the GPU only; there is no CPU path")
        self.act_dtype = torch.bfloat16 if mode == "bfloat16" else torch.float32
        self._buffers: Dict[Any, torch.Tensor] = {}
        self._shared: Dict[Any, Any] = {}
        self.scratch_generation = 0      # bumped when the buffers are dropped (captured graphs go stale)
        self.configure(max_rows, page_size, max_logit_rows)

    def configure(self, max_rows: int, page_size: int, max_logit_rows: int | None = None) -> None:
        """Set the step size limits; existing scratch buffers are dropped."""
        self.max_rows = int(max_rows)
        self.page_size = int(page_size)
        self.max_logit_rows = int(max_logit_rows if max_logit_rows is not None else max_rows)
        self._buffers.clear()
        self.scratch_generation += 1

    @property
    def bf16(self) -> bool:
        return self.mode == "bfloat16"

    def buffer(self, name: str, cols: int, dtype: torch.dtype, rows: int | None = None) -> torch.Tensor:
        """A persistent zero-initialised [rows or max_rows, cols] scratch tensor by name."""
        key = (name, cols, dtype, rows)
        buf = self._buffers.get(key)
        if buf is None:
            buf = torch.zeros((rows if rows is not None else self.max_rows, cols), dtype=dtype, device=self.device)
            self._buffers[key] = buf
        return buf

    def shared(self, key: Any, make: Callable[[], Any]) -> Any:
        """Objects several parts share (one rotary table per distinct parameter set)."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]
