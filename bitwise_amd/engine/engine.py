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

from ..cache.manager import CacheManager, GroupSpec
from ..config.engine import EngineConfig, SamplingParams
from ..sampling.rng import FINGERPRINT_BASIS
from .batch import Segment
from .scheduler import Scheduler, Sequence, Work


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
                                  max_logit_rows=max_logit_rows, use_graphs=config.use_graphs)
        self.sampler = Sampler(rt.device, max_logit_rows)
        self.group_specs = [GroupSpec(g.window) for g in asm.group_specs]
        self.has_state = bool(asm.state_specs)
        self.vocab_size = asm.spec.vocab_size
        self.eos_token_id = asm.spec.eos_token_id

    def reset_slot(self, slot: int) -> None:
        self.storage.reset_slot(slot)

    fused_sampling = True      # run() takes the sampling parameters and may sample inside the step

    def run(self, segments: Seq[Segment], sampling=None):
        """``sampling`` = (temperatures, seeds, positions) of the rows that will be sampled."""
        if sampling is not None:
            temps, seeds, positions = sampling
            sampling = (np.asarray(temps, np.float32), self.sampler.uniforms(temps, seeds, positions))
        return self.runner.step(segments, sampling)

    def sample(self, logits, temperatures, seeds, positions) -> List[int]:
        done = self.runner.last_sampled
        if done is not None and done.numel() == len(temperatures):      # the step's graph has sampled already
            self.runner.last_sampled = None
            return done.cpu().tolist()
        return self.sampler.sample(logits, temperatures, seeds, positions)

    def fingerprints(self, logits, previous) -> List[int]:
        return self.sampler.fingerprints(logits, previous)


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
                                    self.cfg.max_num_seqs, self.cfg.prefix_caching, self.exec.has_state)
        self.sched = Scheduler(self.manager, self.cfg, on_open=self.exec.reset_slot)
        self._seqs: Dict[int, Sequence] = {}
        self._results: Dict[int, RequestResult] = {}
        self._next_id = 0
        self._stats = EngineStats()
        self._start = time.perf_counter()

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
        return self.sched.idle()

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
        events: List[StepEvent] = []
        self._stats.steps += 1
        plan = self.sched.plan()
        for sid in self.sched.preempted_ids:
            self._results[sid].preemptions += 1
        self._stats.preemptions = self.sched.stats.preemptions
        self._stats.prefix_hit_tokens = self.sched.stats.prefix_hit_tokens
        for sid, hit in self.sched.prefix_hits.items():
            self._results[sid].prefix_cached_tokens += hit
        if not plan:
            return events

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
        t0 = self.now()
        # a draw is keyed by what the request's slot records: its seed, and its position once this step's
        # tokens are in the cache (the number of tokens it holds before the new one, src/engine.cpp:473)
        records = [self.manager.record(w.seq.cache) for w in sampled]
        draw = ([w.seq.params.temperature for w in sampled], [r.seed for r in records],
                [r.position + w.n for r, w in zip(records, sampled)])
        if sampled and getattr(self.exec, "fused_sampling", False):
            logits = self.exec.run(segments, draw)
        else:
            logits = self.exec.run(segments)
        new_tokens: List[int] = []
        prints: List[int] = []
        if sampled:
            new_tokens = self.exec.sample(logits, *draw)
            if self.cfg.fingerprint_logits:
                prints = self.exec.fingerprints(logits, [self._results[w.seq.id].logits_fingerprint for w in sampled])
        self._stats.forward_seconds += self.now() - t0

        cursor = 0
        finished: List[Sequence] = []
        for w in plan:
            s = w.seq
            self.sched.commit(w)
            if w.start + w.n == len(s.tokens):
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
        return events

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
        self.sched.remove(s)
        r = self._results[s.id]
        r.finished = True
        r.cancelled = cancelled
        r.finish = self.now()
