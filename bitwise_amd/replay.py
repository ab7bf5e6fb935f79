"""Replaying given tokens through the engine's own step function and cache manager (the role
of logits_chunked, tests/test_main.cpp:200-217, and of Model.logits, python/bindings.cpp:35-52,
with requests that come, pause and end).  Nothing is sampled."""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .cache.manager import CacheManager, GroupSpec, RequestCache
from .engine.batch import Segment
from .engine.runner import ModelRunner
from .engine.storage import CacheStorage
from .model import Model

MAX_STEP_ROWS = 4096


class Replayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, block_size: int = 16, use_graphs: bool = True,
                 max_live: int = 64, model: Optional[Model] = None, poison_freed_pages: bool = False,
                 fingerprint_logits: bool = False, decode_phases: bool = False):
        """``decode_phases``: EngineConfig.decode_phases.  ``poison_freed_pages``: every page that comes back is filled with NaN at once (a fault finder: what a
        later owner of the page reads before writing it shows up in its logits)."""
        self.model = model if model is not None else Model.load(model_dir, dtype)
        asm = self.model.assembled
        rows = max(64, min(int(max_tokens), MAX_STEP_ROWS))
        pages = (int(max_tokens) + block_size - 1) // block_size
        self.manager = CacheManager([GroupSpec(g.window) for g in asm.group_specs], pages, block_size, max_live,
                                    prefix_caching=False, has_state=bool(asm.state_specs))
        self.storage = CacheStorage(asm, pages, max_live, block_size)
        max_len = min(asm.spec.max_positions, max(int(max_tokens), 1))
        self.runner = ModelRunner(asm, self.storage, max_model_len=max_len, max_rows=rows, max_logit_rows=rows,
                                  use_graphs=use_graphs, decode_phases=decode_phases)
        if poison_freed_pages:
            self.manager.on_free = lambda group, page: self.storage.poison_pages(group, [page])
        self.live: Dict[str, RequestCache] = {}
        # per request, the chained hash of every logits row that was asked for (src/engine.cpp:18-29, :246)
        self.fingerprint_logits = fingerprint_logits
        self.fingerprints: Dict[str, int] = {}
        self._sampler = None

    def step(self, entries: Sequence[dict], end: Sequence[str] = ()) -> Optional[np.ndarray]:
        """Run one step; returns the wanted logits [wanted, vocab] or None."""
        segments: List[Segment] = []
        touched: List[RequestCache] = []
        for e in entries:
            rid, toks = str(e["id"]), list(e["tokens"])
            rc = self.live.get(rid)
            if rc is None:
                rc = self.manager.open()
                if rc is None:
                    raise RuntimeError("more live requests than state slots")
                self.storage.reset_slot(rc.slot)
                self.live[rid] = rc
            if not toks:
                continue
            if not self.manager.ensure(rc, rc.computed + len(toks)):
                raise RuntimeError(f"out of cache pages at request {rid}: --max-tokens is too small for this trace")
            want = [int(w) for w in e.get("want", [])]
            if any(w < 0 or w >= len(toks) for w in want):
                raise ValueError(f"request {rid}: 'want' names a place outside its tokens")
            segments.append(Segment(toks, rc.computed, rc.tables, rc.slot, want))
            touched.append(rc)
        out = None
        if segments:
            owners = [str(e["id"]) for e in entries if e.get("tokens") for _ in e.get("want", [])]
            out = self._run(segments, owners)
            for rc, seg in zip(touched, segments):
                self.manager.advance(rc, (), rc.computed + len(seg.tokens))
        for rid in end:
            rc = self.live.pop(str(rid), None)
            if rc is not None:
                self.manager.close(rc)
        return out

    def _chain_fingerprints(self, logits: torch.Tensor, owners: Sequence[str]) -> None:
        """Chain each owner's fingerprint over its rows of ``logits`` in order: the k-th rows of all requests
        are hashed by one launch."""
        from .sampling.rng import FINGERPRINT_BASIS
        from .sampling.sampler import Sampler
        if self._sampler is None:
            self._sampler = Sampler(logits.device, self.runner.max_logit_rows)
        waves: List[List[int]] = []
        seen: Dict[str, int] = {}
        for row, rid in enumerate(owners):
            k = seen.get(rid, 0)
            seen[rid] = k + 1
            if k == len(waves):
                waves.append([])
            waves[k].append(row)
        for rows in waves:
            idx = torch.as_tensor(rows, dtype=torch.long, device=logits.device)
            prev = [self.fingerprints.get(owners[r], FINGERPRINT_BASIS) for r in rows]
            for r, h in zip(rows, self._sampler.fingerprints(logits.index_select(0, idx).contiguous(), prev)):
                self.fingerprints[owners[r]] = h

    def _run(self, segments: List[Segment], owners: Sequence[str] = ()) -> Optional[np.ndarray]:
        limit = self.runner.max_rows
        if sum(len(s.tokens) for s in segments) <= limit:
            lg = self.runner.step(segments)
            if lg is not None and self.fingerprint_logits:
                self._chain_fingerprints(lg, owners)
            return None if lg is None else lg.cpu().numpy()
        # A step larger than the scratch buffers runs as several launches of the step
        # function; the logits do not depend on the cut.
        outs, batch, rows = [], [], 0
        done = [0]

        def flush():
            nonlocal batch, rows
            if batch:
                lg = self.runner.step(batch)
                if lg is not None:
                    if self.fingerprint_logits:
                        self._chain_fingerprints(lg, owners[done[0]:done[0] + lg.shape[0]])
                    done[0] += lg.shape[0]
                    outs.append(lg.cpu().numpy())
            batch, rows = [], 0

        for s in segments:
            off = 0
            while off < len(s.tokens):
                take = min(len(s.tokens) - off, limit - rows)
                want = [w - off for w in s.want if off <= w < off + take]
                batch.append(Segment(s.tokens[off:off + take], s.pos0 + off, s.tables, s.slot, want))
                rows += take
                off += take
                if rows == limit:
                    flush()
        flush()
        return np.concatenate(outs) if outs else None
