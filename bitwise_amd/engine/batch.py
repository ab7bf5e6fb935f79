"""One step's batch as the parts see it: flat rows of several requests (portions of prompts
beside single decoded tokens), with positions, the request each row belongs to, block tables
per cache group, state slots and the rows whose logits are wanted (the reference's BatchRow
list, src/model.h:78-85, turned into device arrays), together with what belongs to the engine
that runs the step: its workspace and its layer calls bound to its caches."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Optional, Sequence

import numpy as np
import torch


@dataclass
class Segment:
    """The next tokens of one request in this step."""
    tokens: Sequence[int]
    pos0: int                          # position of tokens[0]
    tables: Sequence[Sequence[int]]    # per cache group: the request's block table
    slot: int = 0                      # the request's state slot
    want: Sequence[int] = ()           # offsets into ``tokens`` whose logits are wanted


class StepContext:
    """Device arrays of one step.  Rows of a request are contiguous and in position order.  The requests' rows lie
    in an order of the step's own (``segments`` and every per-request array follow it): portions of whole blocks of 16
    rows first, then the other portions, the longest first, then single tokens.  The kernels work on blocks of 16
    rows, and a block that is 16 consecutive tokens of one request from a page's first slot on is one page: a single
    token in front of a long portion would shift every block of it across two pages.  The wanted rows keep the
    order in which the caller gave the requests and their ``want``.

    ``ws``: the workspace of the engine that runs the step (scratch buffers, page size, limits).
    ``calls``: the model's layer calls bound to that engine's caches and state.  ``num_pages``:
    the size of the engine's page pools; a block table that names a page outside is refused
    here, on the host, since the cache writes do not clamp.  A part may keep what it derives
    from the step's shape (tile lists and the like) with ``memo`` for its other layers.
    """

    def __init__(self, segments: Sequence[Segment], num_groups: int, ws, calls: Sequence[Any] = (),
                 num_pages: Optional[int] = None):
        given = list(segments)

        def rank(i: int):
            n = len(given[i].tokens)
            return (2, 0, i) if n == 1 else ((0, 0, i) if n % 16 == 0 else (1, -n, i))
        order = sorted(range(len(given)), key=rank)
        self.segments = [given[i] for i in order]
        self.ws = ws
        self.calls = list(calls)
        self.device = device = ws.device
        self.page_size = ws.page_size
        nseq = len(self.segments)
        rows = sum(len(s.tokens) for s in self.segments)
        self.rows, self.nseq = rows, nseq
        tokens = np.empty(rows, np.int32)
        positions = np.empty(rows, np.int32)
        row_seq = np.empty(rows, np.int32)
        self.seq_start: List[int] = []
        r = 0
        for i, s in enumerate(self.segments):
            n = len(s.tokens)
            self.seq_start.append(r)
            tokens[r:r + n] = s.tokens
            positions[r:r + n] = np.arange(s.pos0, s.pos0 + n, dtype=np.int32)
            row_seq[r:r + n] = i
            r += n
        first_row = {g: self.seq_start[k] for k, g in enumerate(order)}
        want: List[int] = [first_row[g] + w for g, s in enumerate(given) for w in s.want]
        self.num_wanted = len(want)
        widths = [max((len(s.tables[g]) for s in self.segments), default=1) or 1 for g in range(num_groups)]
        tables = []
        for g in range(num_groups):
            t = np.zeros((nseq, widths[g]), np.int32)
            for i, s in enumerate(self.segments):
                row = np.asarray(s.tables[g], np.int32)
                if num_pages is not None and row.size and int(row.max()) >= num_pages:
                    raise ValueError(f"a block table names page {int(row.max())}, the pool has {num_pages}")
                t[i, :len(row)] = np.maximum(row, 0)      # pages given back (-1) are never read
            tables.append(t)
        slots = np.asarray([s.slot for s in self.segments], np.int32)
        parts = [tokens, positions, row_seq, np.asarray(want, np.int32), slots] + [t.reshape(-1) for t in tables]
        packed = torch.from_numpy(np.concatenate(parts)).to(device)
        cuts = np.cumsum([0] + [p.size for p in parts])
        view = [packed[cuts[i]:cuts[i + 1]] for i in range(len(parts))]
        self.tokens, self.positions, self.row_seq, self.want_rows, self.slots = view[:5]
        self.block_tables = [view[5 + g].view(nseq, widths[g]) for g in range(num_groups)]
        self.host_positions = positions
        self._memo: Dict[Any, Any] = {}

    def memo(self, key: Any, make: Callable[[], Any]) -> Any:
        """``make()`` once per step and key."""
        if key not in self._memo:
            self._memo[key] = make()
        return self._memo[key]
