"""The step function: run one batch of (request, its next tokens) through the model, from
the cache that earlier steps left, and return the logits at the wanted places.

It runs only the tokens it is given.  Batches of nothing but single decoded tokens are
replayed from HIP graphs captured per batch-size bucket (the launch sequence of a decode
step is fixed; only the contents of the index arrays change); every other batch is launched
kernel by kernel.  Both routes run the same kernels on the same data layout, so the logits
of a position do not depend on the route.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..csrc import ops
from ..models.assembled import AssembledModel
from .batch import AttentionPlan, Segment, StepContext
from .storage import CacheStorage

GRAPH_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128, 256)


class _StaticDecodeContext:
    """Fixed device arrays for a decode batch of up to ``size`` requests, one row each: the
    step's index arrays and, for sampling inside the graph, each row's temperature and
    uniform.  All of them are views of one device buffer that a step refreshes with a single
    copy from pinned host memory."""

    def __init__(self, size: int, num_groups: int, max_pages: int, device: torch.device):
        self.rows = self.nseq = self.num_wanted = size
        self.device = device
        self.max_pages = max_pages
        off_temp = 3 * size + num_groups * size * max_pages
        off_uni = off_temp + size + ((off_temp + size) & 1)        # 64-bit values start at an even word
        words = off_uni + 2 * size
        self._host = torch.zeros(words, dtype=torch.int32, pin_memory=True)
        self._host_np = self._host.numpy()
        self._dev = torch.zeros(words, dtype=torch.int32, device=device)
        self.tokens = self._dev[0:size]
        self.positions = self._dev[size:2 * size]
        self.slots = self._dev[2 * size:3 * size]
        self.block_tables = [self._dev[3 * size + g * size * max_pages:3 * size + (g + 1) * size * max_pages].view(size, max_pages)
                             for g in range(num_groups)]
        self.temps = self._dev[off_temp:off_temp + size].view(torch.float32)
        self.unis = self._dev[off_uni:off_uni + 2 * size].view(torch.float64)
        self._host_temps = self._host_np[off_temp:off_temp + size].view(np.float32)
        self._host_unis = self._host_np[off_uni:off_uni + 2 * size].view(np.float64)
        self.sampled = torch.zeros(size, dtype=torch.int32, device=device)
        self.row_seq = torch.arange(size, dtype=torch.int32, device=device)
        self.want_rows = torch.arange(size, dtype=torch.int32, device=device)
        self.wants_every_row = True                      # row i is wanted place i: the model need not gather
        self._plan = AttentionPlan(None, 0, None, size)      # implicit tiles: tile t = row t of request t
        self.segments: List[Segment] = []
        # what the host copy of each block-table row was last filled from: (the request's list, its length then);
        # a request's list only grows at its end from step to step, so mostly there is nothing or one entry to write
        self._row_source = [[(None, 0)] * size for _ in range(num_groups)]

    def attention_plan(self, tokens_per_tile: int, group_tiles: int = 1) -> AttentionPlan:
        return self._plan

    def fill(self, segments: Sequence[Segment], sampling=None) -> None:
        """``sampling``: (temperatures, uniforms) of the rows, or None (greedy everywhere)."""
        size, n = self.rows, len(segments)
        self._host_temps[:] = 0.0
        self._host_unis[:] = 0.0
        if sampling is not None:
            self._host_temps[:n] = sampling[0]
            self._host_unis[:n] = sampling[1]
        self.segments = list(segments)
        h = self._host_np
        h[0:size] = -1                      # padding rows: token -1, position -1
        h[size:2 * size] = -1
        h[2 * size:3 * size] = 0
        for i, s in enumerate(segments):
            h[i], h[size + i], h[2 * size + i] = s.tokens[0], s.pos0, s.slot
        base = 3 * size
        for g in range(len(self.block_tables)):
            t = h[base + g * size * self.max_pages:base + (g + 1) * size * self.max_pages].reshape(size, self.max_pages)
            source = self._row_source[g]
            for i, s in enumerate(segments):
                row = s.tables[g]
                was, had = source[i]
                if was is row and had <= len(row):
                    lo = had                        # the same request as last step: only what it got since
                else:
                    lo = 0
                if lo < len(row):
                    # pages given back (-1; outside the window, never read) become 0: any valid page number
                    t[i, lo:len(row)] = [p if p > 0 else 0 for p in row[lo:]]
                    source[i] = (row, len(row))
        self._dev.copy_(self._host, non_blocking=True)


class ModelRunner:
    def __init__(self, model: AssembledModel, storage: CacheStorage, max_model_len: int, use_graphs: bool = True):
        self.model, self.storage = model, storage
        self.rt = model.rt
        self.max_model_len = int(max_model_len)
        self.use_graphs = bool(use_graphs) and model.graph_safe
        self._graphs: Dict[int, tuple] = {}
        self._graph_generation = -1
        self.last_sampled: Optional[torch.Tensor] = None   # tokens the last step's graph sampled, if it did

    # ------------------------------------------------------------------ the step function
    def step(self, segments: Sequence[Segment], sampling=None) -> Optional[torch.Tensor]:
        """Logits [wanted, vocab] (32-bit, on the device, valid until the next step) at the
        wanted places in the order of the segments and of their ``want``; None if none.

        ``sampling`` = (temperatures, uniforms), one per wanted place: a step that is replayed
        from a graph then also samples inside the graph (the same kernel a separate call
        would run) and leaves the tokens in ``last_sampled``; any other step leaves None there."""
        self.last_sampled = None
        if not segments:
            return None
        rows = sum(len(s.tokens) for s in segments)
        wanted = sum(len(s.want) for s in segments)
        if rows > self.rt.max_rows:
            raise ValueError(f"a step of {rows} tokens exceeds the engine's {self.rt.max_rows}")
        if wanted > self.rt.max_logit_rows:
            raise ValueError(f"logits wanted at {wanted} places, the engine allows {self.rt.max_logit_rows}")
        for s in segments:
            if not len(s.tokens):
                raise ValueError("a request without tokens in a step")
            if s.pos0 + len(s.tokens) > self.max_model_len:
                raise ValueError(f"position {s.pos0 + len(s.tokens) - 1} is beyond the model length {self.max_model_len}")
            need = (s.pos0 + len(s.tokens) + self.rt.page_size - 1) // self.rt.page_size
            for t in s.tables:
                if len(t) < need:
                    raise ValueError("a request's block table does not cover its positions")
        decode_only = all(len(s.tokens) == 1 and tuple(s.want) == (0,) for s in segments)
        if self.use_graphs and decode_only and len(segments) <= GRAPH_BUCKETS[-1]:
            return self._step_graph(segments, sampling)
        ctx = StepContext(segments, len(self.model.group_specs), self.rt.device)
        return self.model.forward(ctx)

    # ------------------------------------------------------------------ graph replay
    def _step_graph(self, segments: Sequence[Segment], sampling=None) -> torch.Tensor:
        n = len(segments)
        bucket = next(b for b in GRAPH_BUCKETS if b >= n)
        if bucket > self.rt.max_rows or bucket > self.rt.max_logit_rows:
            ctx = StepContext(segments, len(self.model.group_specs), self.rt.device)
            return self.model.forward(ctx)
        if self._graph_generation != self.rt.scratch_generation:
            self._graphs.clear()                      # a scratch tensor moved: old captures are stale
        entry = self._graphs.get(bucket)
        if entry is None:
            entry = self._capture(bucket, segments)
        ctx, graph, logits = entry
        ctx.fill(segments, sampling)
        graph.replay()
        if sampling is not None:
            self.last_sampled = ctx.sampled[:n]
        return logits[:n]

    def _capture(self, bucket: int, segments: Sequence[Segment]):
        rt = self.rt
        max_pages = (self.max_model_len + rt.page_size - 1) // rt.page_size
        ctx = _StaticDecodeContext(bucket, len(self.model.group_specs), max_pages, rt.device)
        ctx.fill(segments)
        # One eager run first: it creates every scratch buffer the capture will use and it is
        # the step's real work (writing the same cache slots twice with the same values is harmless).
        self.model.forward(ctx)
        torch.cuda.synchronize(rt.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model.forward(ctx)
            ops.sample(logits, bucket, ctx.temps, ctx.unis, ctx.sampled)
        self._graph_generation = rt.scratch_generation
        entry = (ctx, graph, logits)
        self._graphs[bucket] = entry
        return entry
