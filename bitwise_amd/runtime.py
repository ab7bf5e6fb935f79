"""What parts see of the device: the model-wide ``Runtime`` (device, precision mode, objects
that parts share) and the per-engine ``Workspace`` (step size limits, page size and the scratch
buffers of one step function)."""

from __future__ import annotations

from typing import Any, Callable, Dict

import torch

MODES = ("bfloat16", "float32")


class Runtime:
    """Device and precision mode of one model instance, and objects its parts share.

    mode "bfloat16": the kernels and precisions of serving (bfloat16 operands on the matrix
    cores, 32-bit accumulation, 32-bit residual stream, bfloat16 cache).  mode "float32":
    everything in true 32-bit with plain fused multiply-adds.  Nothing here belongs to a
    particular engine: any number of step functions may run one model.
    """

    def __init__(self, mode: str = "bfloat16", device: str | torch.device | None = "cuda:0"):
        if mode not in MODES:
            raise ValueError(f"dtype must be one of {MODES}, got {mode!r}")
        self.mode = mode
        # device None: the model is only described (tensor names and shapes), nothing can run
        self.device = None if device is None else torch.device(device)
        if self.device is not None and self.device.type != "cuda":
            raise RuntimeError("bitwise_amd runs on the GPU only; there is no CPU path")
        self.act_dtype = torch.bfloat16 if mode == "bfloat16" else torch.float32
        self._shared: Dict[Any, Any] = {}

    @property
    def bf16(self) -> bool:
        return self.mode == "bfloat16"

    def shared(self, key: Any, make: Callable[[], Any]) -> Any:
        """Objects several parts share (one rotary table per distinct parameter set)."""
        if key not in self._shared:
            self._shared[key] = make()
        return self._shared[key]


class Workspace:
    """Scratch memory and size limits of one step function (one engine, one replayer, one
    ``Model.logits`` call).  Buffers are made once per name for ``max_rows`` rows and never
    move, so HIP graphs captured over them stay valid; two workspaces share nothing."""

    def __init__(self, device: torch.device, max_rows: int, page_size: int, max_logit_rows: int | None = None,
                 max_table_width: int | None = None):
        self.device = torch.device(device)
        self.max_rows = int(max_rows)
        self.page_size = int(page_size)
        self.max_logit_rows = int(max_logit_rows if max_logit_rows is not None else max_rows)
        # the widest block table a step of this engine can bring (pages of its longest request), if the owner
        # knows it: a part that sizes scratch by the table's width asks once for the widest, not once per width
        self.max_table_width = None if max_table_width is None else int(max_table_width)
        if self.max_rows < 1 or self.max_logit_rows < 1:
            raise ValueError("a workspace needs room for at least one row")
        if self.page_size < 1 or self.page_size & (self.page_size - 1):
            raise ValueError(f"page size must be a power of two, got {self.page_size}")
        self._buffers: Dict[Any, torch.Tensor] = {}
        self.notes: Dict[Any, Any] = {}       # what parts have worked out for this workspace (sizes of their scratch)

    def buffer(self, name: str, cols: int, dtype: torch.dtype, rows: int | None = None) -> torch.Tensor:
        """A persistent zero-initialised [rows or max_rows, cols] scratch tensor by name."""
        key = (name, cols, dtype, rows)
        buf = self._buffers.get(key)
        if buf is None:
            buf = torch.zeros((rows if rows is not None else self.max_rows, cols), dtype=dtype, device=self.device)
            self._buffers[key] = buf
        return buf

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._buffers.values())
