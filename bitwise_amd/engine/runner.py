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
from ..runtime import Workspace
from .batch import Segment, StepContext
from .storage import CacheStorage

GRAPH_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128, 256)
CHAIN_MAX_ROWS = 16       # the graph buckets whose products can run as phases of one launch (ops.chain)


class _StaticDecodeContext:
    """Fixed device arrays for a decode batch of up to ``size`` requests, one row each: the
    step's index arrays and, for sampling inside the graph, each row's temperature and
    uniform.  All of them are views of one device buffer that a step refreshes with a single
    copy from pinned host memory.  Rows beyond the step's requests are padding: token -1,
    position -1, slot -1; every kernel skips a row with a negative position, and a mixer
    with per-request state must skip a row with a negative position or slot."""

    one_row_per_request = True                           # row t is the one token of request t
    wants_every_row = True                               # row i is wanted place i: the model need not gather

    def __init__(self, size: int, num_groups: int, max_pages: int, ws: Workspace, calls, num_pages: int):
        self.rows = self.nseq = self.num_wanted = size
        self.ws, self.calls = ws, list(calls)
        self.device = device = ws.device
        self.page_size = ws.page_size
        self.max_pages = max_pages
        self.num_pages = num_pages
        off_temp = 3 * size + num_groups * size * max_pages
        off_uni = off_temp + size + ((off_temp + size) & 1)        # 64-bit values start at an even word
        words = off_uni + 2 * size
        self._host = torch.zeros(words, dtype=torch.int32, pin_memory=True)
        self._host_np = self._host.numpy()
        self._dev = torch.zeros(words, dtype=torch.int32, device=device)
        self._copied = torch.cuda.Event()                # the last copy out of the pinned buffer
        self._copy_pending = False
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
        # a row whose token id is TOKEN_FROM_FEEDBACK takes the token this graph's last replay sampled for the
        # row: the next step of the same requests in the same order can be launched before the host has the tokens
        self.token_feedback = self.sampled
        self.row_seq = torch.arange(size, dtype=torch.int32, device=device)
        self.want_rows = torch.arange(size, dtype=torch.int32, device=device)
        self.segments: List[Segment] = []
        self.seq_start = list(range(size))
        self._memo: Dict = {}
        # what the host copy of each block-table row was last filled from: (the request's list, its length then);
        # a request's list only grows at its end from step to step, so mostly there is nothing or one entry to write
        self._row_source = [[(None, 0)] * size for _ in range(num_groups)]

    def memo(self, key, make):
        if key not in self._memo:
            self._memo[key] = make()
        return self._memo[key]

    def fill(self, segments: Sequence[Segment], sampling=None) -> None:
        """``sampling``: (temperatures, uniforms) of the rows, or None (greedy everywhere)."""
        if self._copy_pending:
            self._copied.synchronize()      # the pinned buffer is rewritten below: the last copy must have read it
            self._copy_pending = False
        size, n = self.rows, len(segments)
        self._host_temps[:] = 0.0
        self._host_unis[:] = 0.0
        if sampling is not None:
            self._host_temps[:n] = sampling[0]
            self._host_unis[:n] = sampling[1]
        self.segments = list(segments)
        h = self._host_np
        h[0:3 * size] = -1                  # padding rows: token -1, position -1, slot -1
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
                    fresh = row[lo:]
                    if max(fresh) >= self.num_pages:
                        raise ValueError(f"a block table names page {max(fresh)}, the pool has {self.num_pages}")
                    # pages given back (-1; outside the window, never read) become 0: any valid page number
                    t[i, lo:len(row)] = [p if p > 0 else 0 for p in fresh]
                    source[i] = (row, len(row))
        self._dev.copy_(self._host, non_blocking=True)
        self._copied.record()
        self._copy_pending = True


class ModelRunner:
    """The step function of one engine over one model: it owns the workspace (scratch buffers
    sized for ``max_rows`` tokens a step and ``max_logit_rows`` wanted places) and runs on the
    storage's caches.  It keeps nothing in the model, so several runners may share one."""

    def __init__(self, model: AssembledModel, storage: CacheStorage, max_model_len: int, max_rows: int = 256,
                 max_logit_rows: Optional[int] = None, use_graphs: bool = True, decode_phases: bool = False):
        self.model, self.storage = model, storage
        self.rt = model.rt
        self.use_graphs = bool(use_graphs) and model.graph_safe
        # the limits a step is checked against are the caller's; the workspace holds the rows of the graph bucket
        # above them, so that a step of that many decoded tokens still replays a graph (48 requests: the bucket of 64)
        self.max_rows = int(max_rows)
        self.max_logit_rows = int(max_logit_rows if max_logit_rows is not None else max_rows)
        ws_rows, ws_logit_rows = self.max_rows, self.max_logit_rows
        if self.use_graphs:
            bucket = next((b for b in GRAPH_BUCKETS if b >= min(self.max_rows, self.max_logit_rows)), None)
            if bucket is not None:
                ws_rows, ws_logit_rows = max(ws_rows, bucket), max(ws_logit_rows, bucket)
        self.max_model_len = min(int(max_model_len), model.spec.max_positions)
        self.ws = Workspace(model.rt.device, ws_rows, storage.page_size, ws_logit_rows,
                            max_table_width=(self.max_model_len + storage.page_size - 1) // storage.page_size)
        self._graphs: Dict[int, tuple] = {}
        # decode_phases: captured decode steps of few rows in bfloat16 mode run their products as phases of a few
        # launches (ops.chain), if every part launches through ops: the words the phases meet in, and the word that
        # says that a wait inside a launch gave up.
        self.chain_rows = CHAIN_MAX_ROWS if (decode_phases and self.use_graphs and model.rt.bf16 and model.launches_through_ops) else 0
        self.chain_sync = self.chain_err = None
        if self.chain_rows:
            self.chain_sync = torch.zeros(ops.chain_sync_words(), dtype=torch.int32, device=model.rt.device)
            self.chain_err = torch.zeros(1, dtype=torch.int32, device=model.rt.device)
        self.last_sampled: Optional[torch.Tensor] = None   # tokens the last step's graph sampled, if it did
        self.last_graph_rows = 0      # requests of the last step if it was replayed from a graph, else 0

    # ------------------------------------------------------------------ the step function
    def step(self, segments: Sequence[Segment], sampling=None) -> Optional[torch.Tensor]:
        """Logits [wanted, vocab] (32-bit, on the device, valid until the next step) at the
        wanted places in the order of the segments and of their ``want``; None if none.

        ``sampling`` = (temperatures, uniforms), one per wanted place: a step that is replayed
        from a graph then also samples inside the graph (the same kernel a separate call
        would run) and leaves the tokens in ``last_sampled``; any other step leaves None there."""
        self.last_sampled = None
        self.last_graph_rows = 0
        if not segments:
            return None
        rows = sum(len(s.tokens) for s in segments)
        wanted = sum(len(s.want) for s in segments)
        if rows > self.max_rows:
            raise ValueError(f"a step of {rows} tokens exceeds the engine's {self.max_rows}")
        if wanted > self.max_logit_rows:
            raise ValueError(f"logits wanted at {wanted} places, the engine allows {self.max_logit_rows}")
        for s in segments:
            if not len(s.tokens):
                raise ValueError("a request without tokens in a step")
            if s.pos0 + len(s.tokens) > self.max_model_len:
                raise ValueError(f"position {s.pos0 + len(s.tokens) - 1} is beyond the model length {self.max_model_len}")
            need = (s.pos0 + len(s.tokens) + self.ws.page_size - 1) // self.ws.page_size
            for t in s.tables:
                if len(t) < need:
                    raise ValueError("a request's block table does not cover its positions")
        decode_only = all(len(s.tokens) == 1 and tuple(s.want) == (0,) for s in segments)
        if self.use_graphs and decode_only and len(segments) <= GRAPH_BUCKETS[-1]:
            return self._step_graph(segments, sampling)
        return self.model.forward(self._context(segments))

    def _context(self, segments: Sequence[Segment]) -> StepContext:
        return StepContext(segments, len(self.model.group_specs), self.ws, self.storage.bindings, self.storage.num_pages)

    def check_phases(self, bits: Optional[int] = None) -> None:
        """Raise if a wait inside one of the launches of several phases gave up since the last check.  ``bits``: the
        error word as the caller has read it back (None: it is read here, which waits for the device).  The words
        the phases meet in are cleared, so that the next step starts clean."""
        if self.chain_err is None:
            return
        if bits is None:
            bits = int(self.chain_err.item())
        if bits:
            self.chain_sync.zero_()
            self.chain_err.zero_()
            raise RuntimeError(f"a decode step's launch of several phases gave up waiting for a phase (phases {bits:#x}): "
                               "the step's results are void")

    # ------------------------------------------------------------------ graph replay
    def _step_graph(self, segments: Sequence[Segment], sampling=None) -> torch.Tensor:
        n = len(segments)
        bucket = next(b for b in GRAPH_BUCKETS if b >= n)
        if bucket > self.ws.max_rows or bucket > self.ws.max_logit_rows:
            return self.model.forward(self._context(segments))
        entry = self._graphs.get(bucket)
        if entry is None:
            entry = self._capture(bucket)
        ctx, graph, logits = entry
        ctx.fill(segments, sampling)
        graph.replay()
        if sampling is not None:
            self.last_sampled = ctx.sampled[:n]
        self.last_graph_rows = n
        return logits[:n]

    def _capture(self, bucket: int):
        ws = self.ws
        max_pages = (self.max_model_len + ws.page_size - 1) // ws.page_size
        ctx = _StaticDecodeContext(bucket, len(self.model.group_specs), max_pages, ws, self.storage.bindings,
                                   self.storage.num_pages)
        # One eager run first, on rows that are all padding: it creates every scratch buffer the capture
        # will use and touches neither cache nor state (a real step run here and then replayed from the
        # fresh graph would advance a stateful mixer twice).
        def forward():
            # (the warm-up runs what the capture will run: the kernels' one-time set-up happens outside the capture)
            if bucket <= self.chain_rows:
                with ops.chain(self.chain_sync, self.chain_err):
                    return self.model.forward(ctx)
            return self.model.forward(ctx)

        ctx.fill([])
        forward()
        torch.cuda.synchronize(ws.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = forward()
            ops.sample(logits, bucket, ctx.temps, ctx.unis, ctx.sampled)
        entry = (ctx, graph, logits)
        self._graphs[bucket] = entry
        return entry
