"""One step's batch as the parts see it: flat rows of several requests (portions of prompts
beside single decoded tokens), with positions, the request each row belongs to, block tables
per cache group, state slots and the rows whose logits are wanted (the reference's BatchRow
list, src/model.h:78-85, turned into device arrays)."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..parts.attention import DECODE_MIN_CONTEXT


@dataclass
class Segment:
    """The next tokens of one request in this step."""
    tokens: Sequence[int]
    pos0: int                          # position of tokens[0]
    tables: Sequence[Sequence[int]]    # per cache group: the request's block table
    slot: int = 0                      # the request's state slot
    want: Sequence[int] = ()           # offsets into ``tokens`` whose logits are wanted


@dataclass
class AttentionPlan:
    fold_tiles: Optional[torch.Tensor]
    fold_count: int
    decode_tiles: Optional[torch.Tensor]      # None with a positive count: tile t is row t of request t
    decode_count: int


class StepContext:
    """Device arrays of one step.  Rows of a request are contiguous and in position order."""

    def __init__(self, segments: Sequence[Segment], num_groups: int, device: torch.device):
        self.segments = list(segments)
        self.device = device
        nseq = len(self.segments)
        rows = sum(len(s.tokens) for s in self.segments)
        self.rows, self.nseq = rows, nseq
        tokens = np.empty(rows, np.int32)
        positions = np.empty(rows, np.int32)
        row_seq = np.empty(rows, np.int32)
        want: List[int] = []
        self.seq_start: List[int] = []
        r = 0
        for i, s in enumerate(self.segments):
            n = len(s.tokens)
            self.seq_start.append(r)
            tokens[r:r + n] = s.tokens
            positions[r:r + n] = np.arange(s.pos0, s.pos0 + n, dtype=np.int32)
            row_seq[r:r + n] = i
            want.extend(r + w for w in s.want)
            r += n
        self.num_wanted = len(want)
        widths = [max((len(s.tables[g]) for s in self.segments), default=1) or 1 for g in range(num_groups)]
        tables = []
        for g in range(num_groups):
            t = np.zeros((nseq, widths[g]), np.int32)
            for i, s in enumerate(self.segments):
                row = np.asarray(s.tables[g], np.int32)
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
        self._plans: Dict[tuple, AttentionPlan] = {}

    def attention_plan(self, tokens_per_tile: int, group_tiles: int = 1) -> AttentionPlan:
        """Tiles of up to ``tokens_per_tile`` consecutive rows of one request; every request's
        run of tiles is padded with empty tiles to a multiple of ``group_tiles`` (the tiles one
        wave owns must belong to one request).  Single decoded tokens with a long context go
        to the decode kernel (a wave per 64-key partition)."""
        plan = self._plans.get((tokens_per_tile, group_tiles))
        if plan is not None:
            return plan
        fold, split = [], []
        for i, s in enumerate(self.segments):
            n, r0 = len(s.tokens), self.seq_start[i]
            if n == 1 and s.pos0 + 1 >= DECODE_MIN_CONTEXT:
                split.append((r0, 1, i, 0))
                continue
            for off in range(0, n, tokens_per_tile):
                fold.append((r0 + off, min(tokens_per_tile, n - off), i, 0))
            while len(fold) % group_tiles:
                fold.append((r0, 0, i, 0))
        both = np.asarray(fold + split, np.int32).reshape(-1, 4)
        dev = torch.from_numpy(both).to(self.device)
        plan = AttentionPlan(dev[:len(fold)].contiguous() if fold else None, len(fold),
                             dev[len(fold):].contiguous() if split else None, len(split))
        self._plans[(tokens_per_tile, group_tiles)] = plan
        return plan
