"""Choosing tokens from logits rows on the device: greedy (first maximum) for temperature
<= 0, else an inverse-CDF draw from softmax(logits / T) at a counter-based uniform
(src/engine.cpp:40-80, :467-476).  The reference samples with nothing else (no top-k or
top-p, README.md:207).  Also the chained fingerprint of the logits behind every generated
token (src/engine.cpp:18-29, :246)."""

from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from ..csrc import ops
from .rng import STREAM_SAMPLE, counter_uniform


class Sampler:
    def __init__(self, device: torch.device, max_rows: int):
        self.device = device
        self.max_rows = max_rows
        self._temp = torch.zeros(max_rows, dtype=torch.float32, device=device)
        self._uni = torch.zeros(max_rows, dtype=torch.float64, device=device)
        self._out = torch.zeros(max_rows, dtype=torch.int32, device=device)
        self._h_in = torch.zeros(max_rows, dtype=torch.int64, device=device)
        self._h_out = torch.zeros(max_rows, dtype=torch.int64, device=device)

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
               positions: Sequence[int]) -> List[int]:
        """One token per row.  ``positions[r]`` is the number of tokens the request holds
        before the new one: the counter of its random draw (src/engine.cpp:473)."""
        rows = len(temperatures)
        if rows == 0:
            return []
        if rows > self.max_rows or logits.shape[0] < rows:
            raise ValueError("more rows to sample than the sampler was made for")
        return self.sample_on_device(logits, temperatures, self.uniforms(temperatures, seeds, positions)).cpu().tolist()

    def sample_on_device(self, logits: torch.Tensor, temperatures: Sequence[float], uniforms: np.ndarray) -> torch.Tensor:
        """The tokens as a device tensor (a view of the sampler's buffer, valid until its next call)."""
        rows = len(temperatures)
        if rows > self.max_rows or logits.shape[0] < rows:
            raise ValueError("more rows to sample than the sampler was made for")
        self._temp[:rows].copy_(torch.from_numpy(np.asarray(temperatures, np.float32)))
        self._uni[:rows].copy_(torch.from_numpy(np.asarray(uniforms, np.float64)))
        ops.sample(logits, rows, self._temp, self._uni, self._out)
        return self._out[:rows]

    @staticmethod
    def uniforms(temperatures: Sequence[float], seeds: Sequence[int], positions: Sequence[int]) -> np.ndarray:
        """The uniform of each row's draw (0 where the row is greedy)."""
        return np.asarray([counter_uniform(s, p, STREAM_SAMPLE) if t > 0 else 0.0
                           for t, s, p in zip(temperatures, seeds, positions)], np.float64)

    def fingerprints(self, logits: torch.Tensor, previous: Sequence[int]) -> List[int]:
        """previous[r] chained over row r of ``logits`` (unsigned 64-bit values)."""
        rows = len(previous)
        if rows == 0:
            return []
        h = np.asarray(previous, np.uint64).view(np.int64)
        self._h_in[:rows].copy_(torch.from_numpy(h))
        ops.fingerprint(logits, rows, self._h_in, self._h_out)
        return self._h_out[:rows].cpu().numpy().view(np.uint64).tolist()
