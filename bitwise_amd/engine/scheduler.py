"""The scheduler: admits requests, cuts prompts into portions under the step's token budget,
decodes, and decides what happens when pages run out (src/engine.cpp:304-376, :146-237).

It owns no device memory and runs no kernels, so its decisions can be tested on the CPU:
``plan()`` turns the queues and the cache manager's state into this step's work list,
``commit()`` books the tokens a step produced.

Policy, as in the reference:
* running requests first, oldest first (one decode token each, or the rest of an unfinished
  prompt cut to the remaining budget);
* then waiting requests in arrival order, while there are fewer than ``max_num_seqs`` running
  and budget is left; the head of the queue blocks those behind it (no skipping);
* a running request that cannot get its pages preempts the youngest running request that is
  not already scheduled in this step and is not itself; if there is none, it is preempted
  itself.  Preemption gives back all pages and the slot, sets ``computed`` to 0 and puts the
  request back into the waiting queue by id; tokens generated so far are kept and recomputed
  as prompt (recompute preemption);
* a waiting request that cannot get its pages gives back what it took and waits;
* a request whose worst case can never fit is refused at submission.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

from ..cache.manager import CacheManager, RequestCache
from ..config.engine import EngineConfig, Fault, SamplingParams


@dataclass
class Sequence:
    id: int
    tokens: List[int]                 # prompt, then generated tokens
    prompt_len: int
    params: SamplingParams
    cache: Optional[RequestCache] = None      # pages and slot while admitted
    running: bool = False
    done: bool = False

    @property
    def computed(self) -> int:
        return self.cache.computed if self.cache is not None else 0

    def generated(self) -> int:
        return len(self.tokens) - self.prompt_len


@dataclass
class Work:
    seq: Sequence
    n: int                            # tokens of this request in the step
    start: int                        # position of the first of them


@dataclass
class SchedulerStats:
    preemptions: int = 0
    prefix_hit_tokens: int = 0


class Scheduler:
    def __init__(self, manager: CacheManager, config: EngineConfig, on_open=None):
        self.manager = manager
        self.cfg = config
        self.on_open = on_open                  # called with the slot a request has just taken
        self.waiting: List[Sequence] = []       # in id order
        self.running: List[Sequence] = []       # sorted by id
        self.stats = SchedulerStats()
        self.preempted_ids: List[int] = []      # ids preempted during the last plan()
        self.prefix_hits: Dict[int, int] = {}   # id -> tokens served from cached pages in the last plan()

    # ------------------------------------------------------------------ queues
    def submit(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def idle(self) -> bool:
        return not self.running and not self.waiting

    def _requeue(self, seq: Sequence) -> None:
        pos = next((i for i, w in enumerate(self.waiting) if w.id > seq.id), len(self.waiting))
        self.waiting.insert(pos, seq)

    def _drop_cache(self, seq: Sequence) -> None:
        if seq.cache is not None:
            self.manager.close(seq.cache)
            seq.cache = None

    def preempt(self, seq: Sequence) -> None:
        self._drop_cache(seq)
        seq.running = False
        self.running.remove(seq)
        self._requeue(seq)
        self.stats.preemptions += 1
        self.preempted_ids.append(seq.id)

    def remove(self, seq: Sequence, cancelled: bool = False) -> None:
        """Finish or cancel: give back everything and leave the queues."""
        if cancelled and self.cfg.fault == Fault.CANCEL_KEEPS_PAGES and seq.cache is not None:
            seq.cache.tables = [[] for _ in seq.cache.tables]         # (the injected bug: the pages are forgotten)
        self._drop_cache(seq)
        if seq.running:
            self.running.remove(seq)
        elif seq in self.waiting:
            self.waiting.remove(seq)
        seq.running = False
        seq.done = True

    # ------------------------------------------------------------------ one step's decisions
    def _cut(self, s: Sequence, n: int) -> int:
        """The length of a portion of ``s`` that the budget ends after ``n`` tokens, short of the prompt's end: shortened
        to end at a multiple of ``portion_align`` tokens, so that the next portion starts with a page (0: the request
        waits a step, if nothing is left then) -- unless what an exact cut leaves is shorter than that anyway.  Only
        where every step has room for such a portion whatever else runs (the budget exceeds the running requests'
        single tokens by ``portion_align`` at least); else the portion is cut at the budget."""
        a = self.cfg.portion_align
        if a <= 1 or self.cfg.max_batched_tokens - self.cfg.max_num_seqs < a:
            return n
        if len(s.tokens) - s.computed - n < a:
            return n
        end = (s.computed + n) // a * a
        return max(end - s.computed, 0)

    def plan(self) -> List[Work]:
        budget = self.cfg.max_batched_tokens
        plan: List[Work] = []
        scheduled: List[Sequence] = []
        self.preempted_ids = []
        self.prefix_hits = {}

        # 1. running requests, oldest first
        for s in list(self.running):
            if not s.running:
                continue                      # preempted earlier in this loop
            need = len(s.tokens) - s.computed
            n = need
            if n == 0:
                continue
            if n > budget:
                if budget <= 0:
                    continue                  # a decode row without budget waits for the next step
                n = self._cut(s, budget)      # cut the rest of the prompt to the budget
                if n == 0:
                    continue
            ok = self.manager.ensure(s.cache, s.computed + n)
            while not ok:
                victim = next((v for v in reversed(self.running) if v is not s and v not in scheduled), None)
                if victim is None:
                    break
                self.preempt(victim)
                ok = self.manager.ensure(s.cache, s.computed + n)
            if not ok:
                self.preempt(s)
                continue
            plan.append(Work(s, n, s.computed))
            scheduled.append(s)
            budget -= n

        # 2. waiting requests in arrival order
        while self.waiting and len(self.running) < self.cfg.max_num_seqs:
            if budget <= 0:
                break
            s = self.waiting[0]
            if s.cache is None:
                s.cache = self.manager.open(seed=s.params.seed)
                if s.cache is None:
                    break                     # no state slot free (cannot happen while slots == max_num_seqs)
                if self.on_open is not None:
                    self.on_open(s.cache.slot)
            hit = 0
            if not any(s.cache.tables):
                hit = self.manager.admit_prefix(s.cache, s.tokens)
            need = len(s.tokens) - s.computed
            n = need if need <= budget else self._cut(s, budget)
            if n == 0 and need > 0:
                self._drop_cache(s)           # (as below: nothing of this request is held while it waits)
                break
            if not self.manager.ensure(s.cache, s.computed + n):
                self._drop_cache(s)           # the prefix hit is retried at the next attempt
                break
            if hit:
                self.prefix_hits[s.id] = hit
                self.stats.prefix_hit_tokens += hit
            self.waiting.pop(0)
            s.running = True
            pos = next((i for i, r in enumerate(self.running) if r.id > s.id), len(self.running))
            self.running.insert(pos, s)
            if n > 0:
                plan.append(Work(s, n, s.computed))
                budget -= n
        return plan

    def commit(self, work: Work) -> None:
        """The step ran: ``work.n`` more tokens of the request are in the cache."""
        s = work.seq
        self.manager.advance(s.cache, s.tokens, work.start + work.n)
