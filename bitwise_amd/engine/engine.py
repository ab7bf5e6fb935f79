"""The serving engine: continuous batching over the paged cache with chunked prefill, prefix
caching and recompute preemption, with the reference's interface (src/engine.h:96-113):
add_request / cancel / step / idle / result / stats.

A request's tokens depend on nothing but its own prompt and sampling parameters: the kernels
give every position the same logits however the batch was cut, and sampling is keyed by
(seed, position).  ``logits_fingerprint`` chains a hash over the logits row behind every
generated token, so equality of runs can be checked to the last bit.
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence as Seq

import numpy as np
import torch

from ..cache.manager import CacheManager, GroupSpec
from ..config.engine import EngineConfig, Fault, SamplingParams
from ..csrc import ops
from ..sampling.rng import FINGERPRINT_BASIS
from .batch import Segment
from .scheduler import Scheduler, Sequence, Work

AHEAD_TOKEN = -2       # the token id of a row whose token the step before is still choosing (ops.TOKEN_FROM_FEEDBACK)


class _Pending:
    """A step that has been launched: what it will leave in pinned host memory once its event has passed."""

    def __init__(self, n: int, event, tokens_host, prints_host, graph_rows: int, check=None):
        self.n, self.event, self.tokens_host, self.prints_host, self.graph_rows = n, event, tokens_host, prints_host, graph_rows
        self.prints_dev = None
        self.check = check              # called once the device is through: raises if the step's results are void

    def result(self):
        """(tokens, fingerprints or []) of the sampled rows; waits for the device."""
        if self.n == 0:
            return [], []
        self.event.synchronize()
        if self.check is not None:
            self.check()
        tokens = self.tokens_host[:self.n].tolist()
        prints = self.prints_host[:self.n].numpy().view(np.uint64).tolist() if self.prints_host is not None else []
        return tokens, prints


class _Done:
    """The same face for an executor that computes at once (the stand-in device of the scheduler's tests)."""

    def __init__(self, tokens, prints):
        self._r = (tokens, prints)
        self.n = len(tokens)

    def result(self):
        return self._r


@dataclass
class _Flight:
    """One step between its launch and its bookkeeping."""
    plan: List[Work]
    sampled: List[Work]
    pending: object
    t0: float


@dataclass
class RequestResult:
    tokens: List[int] = field(default_factory=list)     # generated tokens
    finished: bool = False
    cancelled: bool = False
    logits_fingerprint: int = FINGERPRINT_BASIS
    preemptions: int = 0
    prefix_cached_tokens: int = 0
    arrival: float = 0.0
    first_token: float = -1.0
    finish: float = -1.0
    token_times: List[float] = field(default_factory=list)


@dataclass
class StepEvent:
    id: int
    tokens: List[int]
    finished: bool


@dataclass
class EngineStats:
    steps: int = 0
    prefill_tokens: int = 0
    decode_rows: int = 0
    generated_tokens: int = 0
    preemptions: int = 0
    prefix_hit_tokens: int = 0
    evictions: int = 0
    forward_seconds: float = 0.0


class GpuExecutor:
    """What the engine needs from the device: run a batch, pick tokens, hash logits rows."""

    def __init__(self, model, config: EngineConfig):
        from ..sampling.sampler import Sampler
        from .runner import ModelRunner
        from .storage import CacheStorage

        asm = model.assembled
        rt = asm.rt
        if rt.mode != config.dtype:
            raise ValueError(f"the model was loaded as {rt.mode}, the engine is configured for {config.dtype}")
        # caches, state, scratch buffers and captured graphs are this executor's own: the model holds
        # weights only, so other engines may run it at the same time
        self.storage = CacheStorage(asm, config.num_blocks, config.max_num_seqs, config.block_size)
        max_len = config.max_model_len or asm.spec.max_positions
        self.max_model_len = min(max_len, asm.spec.max_positions)
        max_logit_rows = min(config.max_num_seqs, config.max_batched_tokens)
        self.runner = ModelRunner(asm, self.storage, self.max_model_len, max_rows=config.max_batched_tokens,
                                  max_logit_rows=max_logit_rows, use_graphs=config.use_graphs,
                                  decode_phases=config.decode_phases)
        self.sampler = Sampler(rt.device, max_logit_rows)
        # two steps may be under way at a time (one being read back, one launched ahead): two sets of buffers
        self._flip = 0
        self._events = [torch.cuda.Event(), torch.cuda.Event()]
        self._tokens_host = [torch.zeros(max_logit_rows, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._phase_err_host = [torch.zeros(1, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._prints_host = [torch.zeros(max_logit_rows, dtype=torch.int64, pin_memory=True) for _ in range(2)]
        self._prints_dev = [torch.zeros(max_logit_rows, dtype=torch.int64, device=rt.device) for _ in range(2)]
        self._prints_in = torch.zeros(max_logit_rows, dtype=torch.int64, device=rt.device)
        self.group_specs = [GroupSpec(g.window) for g in asm.group_specs]
        self.has_state = bool(asm.state_specs)
        self.prefix_reusable = asm.prefix_reusable      # every mixer keeps what it computed in its pages
        self.run_ahead_safe = asm.run_ahead_safe        # no mixer minds a row that runs for a request that has ended
        self.vocab_size = asm.spec.vocab_size
        self.eos_token_id = asm.spec.eos_token_id

    def reset_slot(self, slot: int) -> None:
        self.storage.reset_slot(slot)

    # ------------------------------------------------------------------ one step, launched and read back apart
    def launch(self, segments: Seq[Segment], draw, previous_prints, after: "Optional[_Pending]" = None) -> "_Pending":
        """Run a batch and everything behind it on the device without waiting for any of it: the model,
        the choice of tokens for the rows that end their request's known tokens, their logits fingerprints,
        and the copies of tokens and fingerprints to pinned host memory.  ``draw`` = (temperatures, seeds,
        positions) of those rows.  ``previous_prints``: their fingerprints so far (host integers), or None
        to chain them from ``after``, the step launched just before for the same rows in the same order
        (whose tokens this step also takes on the device)."""
        temps, seeds, positions = draw
        n = len(temps)
        sampling = (np.asarray(temps, np.float32), self.sampler.uniforms(temps, seeds, positions)) if n else None
        logits = self.runner.step(segments, sampling)
        slot = self._flip
        self._flip ^= 1
        pend = _Pending(n, self._events[slot], self._tokens_host[slot], None, self.runner.last_graph_rows)
        if n and self.runner.chain_rows and self.runner.last_graph_rows:
            # the word that says whether a wait inside a launch of several phases gave up comes back with the tokens
            word = self._phase_err_host[slot]
            word.copy_(self.runner.chain_err, non_blocking=True)
            pend.check = lambda: self.runner.check_phases(int(word[0]))
        if n:
            sampled = self.runner.last_sampled
            if sampled is None:
                sampled = self.sampler.sample_on_device(logits, temps, sampling[1])
            pend.tokens_host[:n].copy_(sampled[:n], non_blocking=True)
            if previous_prints is not None or after is not None:
                h_in = self._prints_in
                if previous_prints is not None:
                    h_in[:n].copy_(torch.from_numpy(np.asarray(previous_prints, np.uint64).view(np.int64)))
                else:
                    h_in = after.prints_dev
                pend.prints_dev = self._prints_dev[slot]
                ops.fingerprint(logits, n, h_in, pend.prints_dev)
                pend.prints_host = self._prints_host[slot]
                pend.prints_host[:n].copy_(pend.prints_dev[:n], non_blocking=True)
            pend.event.record()
        return pend

    def can_run_ahead(self, pend: "_Pending", rows: int) -> bool:
        """Whether the next decode step of the same ``rows`` requests may be launched before this one's
        tokens are read: it was replayed from a graph that sampled them (the next replay of that graph finds
        them on the device) and every mixer says that a row may run for a request that has just ended."""
        return pend.graph_rows == rows and pend.n == rows and self.run_ahead_safe

class Engine:
    def __init__(self, target, draft=None, config: Optional[EngineConfig] = None, executor=None):
        """``target``: a Model.  ``draft`` belongs to speculative decoding, which this engine
        does not do; it must be None.  ``executor`` replaces the device (tests of the
        scheduler's decisions pass a stand-in)."""
        if draft is not None:
            raise ValueError("speculative decoding is not part of this engine; pass draft=None")
        self.cfg = config or EngineConfig()
        self.cfg.validate()
        self.exec = executor if executor is not None else GpuExecutor(target, self.cfg)
        self.manager = CacheManager(self.exec.group_specs, self.cfg.num_blocks, self.cfg.block_size,
                                    self.cfg.max_num_seqs, self.cfg.prefix_caching,
                                    not getattr(self.exec, "prefix_reusable", not self.exec.has_state), fault=self.cfg.fault)
        self.sched = Scheduler(self.manager, self.cfg, on_open=self.exec.reset_slot)
        self._seqs: Dict[int, Sequence] = {}
        self._results: Dict[int, RequestResult] = {}
        self._next_id = 0
        self._stats = EngineStats()
        self._start = time.perf_counter()
        self._ahead: Optional[_Flight] = None       # a step launched before the one before it was read back

    # ------------------------------------------------------------------ interface
    def now(self) -> float:
        return time.perf_counter() - self._start

    def add_request(self, prompt: Seq[int], params: Optional[SamplingParams] = None) -> int:
        params = params or SamplingParams()
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError("empty prompt")
        if any(t < 0 or t >= self.exec.vocab_size for t in prompt):
            raise ValueError("token id out of range")
        worst = len(prompt) + params.max_new_tokens + 1
        if not self.manager.can_ever_hold(worst, self.cfg.max_batched_tokens):
            raise ValueError("request can never fit in the KV cache")
        if len(prompt) + params.max_new_tokens > self.exec.max_model_len:
            raise ValueError(f"prompt and new tokens exceed the model length {self.exec.max_model_len}")
        seq = Sequence(self._next_id, prompt, len(prompt), params)
        self._next_id += 1
        self._seqs[seq.id] = seq
        self._results[seq.id] = RequestResult(arrival=self.now())
        self.sched.submit(seq)
        return seq.id

    def cancel(self, id: int) -> None:
        seq = self._seqs.pop(id, None)
        if seq is None or seq.done:
            return
        self._finish(seq, cancelled=True)

    def idle(self) -> bool:
        return self.sched.idle() and (self._ahead is None or all(w.seq.done for w in self._ahead.plan))

    @property
    def num_running(self) -> int:
        return len(self.sched.running)

    @property
    def num_waiting(self) -> int:
        return len(self.sched.waiting)

    @property
    def free_blocks(self) -> int:
        """Free pages of the first cache group (the reference's one pool); all pages if the model keeps no paged cache."""
        return self.manager.free_pages(0) if self.manager.pools else self.cfg.num_blocks

    def result(self, id: int) -> RequestResult:
        return self._results[id]

    @property
    def stats(self) -> EngineStats:
        return self._stats

    @property
    def config(self) -> EngineConfig:
        return self.cfg

    def debug_state(self) -> str:
        lines = [f"free_blocks={self.free_blocks}"]
        for tag, queue in (("running", self.sched.running), ("waiting", self.sched.waiting)):
            for s in queue:
                pages = len(s.cache.tables[0]) if s.cache is not None and s.cache.tables else 0
                lines.append(f"{tag} id={s.id} len={len(s.tokens)} prompt={s.prompt_len} computed={s.computed} "
                             f"blocks={pages} gen={s.generated()}/{s.params.max_new_tokens}")
        return "\n".join(lines) + "\n"

    # ------------------------------------------------------------------ one step
    def step(self) -> List[StepEvent]:
        """One step's tokens.  The step is planned and launched here unless the call before launched it
        ahead; before its tokens are waited for, the next step is launched ahead if it can only be one more
        token for each of the same requests (src/engine.cpp:304-488 is the synchronous form of this)."""
        events: List[StepEvent] = []
        self._stats.steps += 1
        flight, self._ahead = self._ahead, None
        if flight is not None and all(w.seq.done for w in flight.plan):
            flight = None                          # everyone in it has ended or was cancelled meanwhile
        if flight is None:
            flight = self._launch_planned()
            if flight is None:
                return events
        ahead = self._launch_ahead(flight)
        self._complete(flight, events)
        if ahead is not None and any(not w.seq.done for w in ahead.sampled):
            self._ahead = ahead
        return events

    def _launch_planned(self) -> Optional[_Flight]:
        plan = self.sched.plan()
        for sid in self.sched.preempted_ids:
            self._results[sid].preemptions += 1
        self._stats.preemptions = self.sched.stats.preemptions
        self._stats.prefix_hit_tokens = self.sched.stats.prefix_hit_tokens
        for sid, hit in self.sched.prefix_hits.items():
            self._results[sid].prefix_cached_tokens += hit
        if not plan:
            return None
        segments: List[Segment] = []
        sampled: List[Work] = []
        for w in plan:
            s = w.seq
            last = w.start + w.n == len(s.tokens)
            segments.append(Segment(s.tokens[w.start:w.start + w.n], w.start, s.cache.tables, s.cache.slot,
                                    [w.n - 1] if last else []))
            if last:
                sampled.append(w)
            if w.n == 1 and last and s.generated() > 0:
                self._stats.decode_rows += 1
            else:
                self._stats.prefill_tokens += w.n
        # a draw is keyed by what the request's slot records: its seed, and its position once this step's
        # tokens are in the cache (the number of tokens it holds before the new one, src/engine.cpp:473)
        records = [self.manager.record(w.seq.cache) for w in sampled]
        draw = ([w.seq.params.temperature for w in sampled], [r.seed for r in records],
                [r.position + w.n for r, w in zip(records, sampled)])
        if self.cfg.fault == Fault.RNG_KEYED_BY_STEP:
            draw = (draw[0], draw[1], [self._stats.steps] * len(sampled))
        prints = [self._results[w.seq.id].logits_fingerprint for w in sampled] if self.cfg.fingerprint_logits else None
        t0 = self.now()
        return _Flight(plan, sampled, self._exec_launch(segments, draw, prints), t0)

    def _exec_launch(self, segments, draw, prints):
        if hasattr(self.exec, "launch"):
            return self.exec.launch(segments, draw, prints)
        logits = self.exec.run(segments)                       # an executor that computes at once
        tokens = self.exec.sample(logits, *draw) if draw[0] else []
        return _Done(tokens, self.exec.fingerprints(logits, prints) if prints is not None and draw[0] else [])

    def _launch_ahead(self, flight: _Flight) -> Optional[_Flight]:
        """The step after ``flight``, launched before ``flight``'s tokens are known, if it is certain what it
        is up to the tokens themselves: ``flight`` decodes one token for every running request, nobody
        waits, nobody reaches its length, and every request gets its next page without taking one from
        another.  A request that turns out to have ended with ``flight``'s token (end of sequence, a
        cancellation) has its row of this step thrown away; the other rows do not depend on it."""
        cfg, ex = self.cfg, self.exec
        running = self.sched.running
        if not (cfg.run_ahead and getattr(ex, "can_run_ahead", None) and not self.sched.waiting):
            return None
        if len(flight.plan) != len(running) or len(flight.sampled) != len(running):
            return None
        if not all(w.n == 1 and w.seq is s for w, s in zip(flight.plan, running)):
            return None
        if not ex.can_run_ahead(flight.pending, len(running)):
            return None
        for s in running:
            if s.generated() + 2 > s.params.max_new_tokens or len(s.tokens) + 2 > ex.max_model_len:
                return None                 # it ends with this step's token, or with the next: the plain path
        if sum(self.manager.pages_missing(s.cache, len(s.tokens) + 1) for s in running) > self.manager.free_pages_least():
            return None
        for s in running:
            if not self.manager.ensure(s.cache, len(s.tokens) + 1):
                return None                 # (pages taken so far stay with their requests)
        plan = [Work(s, 1, len(s.tokens)) for s in running]
        segments = [Segment([AHEAD_TOKEN], len(s.tokens), s.cache.tables, s.cache.slot, [0]) for s in running]
        records = [self.manager.record(s.cache) for s in running]
        draw = ([s.params.temperature for s in running], [r.seed for r in records], [len(s.tokens) + 1 for s in running])
        if cfg.fault == Fault.RNG_KEYED_BY_STEP:
            draw = (draw[0], draw[1], [self._stats.steps + 1] * len(running))
        t0 = self.now()
        pending = ex.launch(segments, draw, None, after=flight.pending if cfg.fingerprint_logits else None)
        self._stats.decode_rows += len(running)
        return _Flight(plan, list(plan), pending, t0)

    def _complete(self, flight: _Flight, events: List[StepEvent]) -> None:
        new_tokens, prints = flight.pending.result()
        self._stats.forward_seconds += self.now() - flight.t0
        cursor = 0
        finished: List[Sequence] = []
        chosen = {id(w) for w in flight.sampled}
        for w in flight.plan:
            s = w.seq
            last = id(w) in chosen
            if s.done:                                 # ended or cancelled since the launch: the row is thrown away
                cursor += 1 if last else 0
                continue
            self.sched.commit(w)
            if last:
                token = new_tokens[cursor]
                if prints:
                    self._results[s.id].logits_fingerprint = prints[cursor]
                cursor += 1
                if self._append(s, token, events):
                    finished.append(s)
        for s in finished:
            self._finish(s, cancelled=False)
            self._seqs.pop(s.id, None)
        self._stats.evictions = self.manager.evictions

    # ------------------------------------------------------------------ bookkeeping
    def _append(self, s: Sequence, token: int, events: List[StepEvent]) -> bool:
        """Stop rules of src/engine.cpp:250-254; the end-of-sequence token is kept."""
        r = self._results[s.id]
        s.tokens.append(token)
        r.tokens.append(token)
        t = self.now()
        if r.first_token < 0:
            r.first_token = t
        r.token_times.append(t)
        self._stats.generated_tokens += 1
        events.append(StepEvent(s.id, [token], False))
        eos = (not s.params.ignore_eos) and token == self.exec.eos_token_id
        if eos or s.generated() >= s.params.max_new_tokens:
            events[-1].finished = True
            return True
        return False

    def _finish(self, s: Sequence, cancelled: bool) -> None:
        self.sched.remove(s, cancelled)
        r = self._results[s.id]
        r.finished = True
        r.cancelled = cancelled
        r.finish = self.now()
