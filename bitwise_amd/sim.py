"""Randomized scheduling traces against a solo-run oracle, after the reference's simulator
(sim/simulate.cpp:81-217): seeded workloads with shared and repeated prompts, greedy and
sampled decoding, staggered arrivals, cancellations, and an engine configuration drawn at
random (a cache small enough to force preemption, budgets small enough to force chunked
prompts, prefix caching on or off).  Every request that was not cancelled must produce the
tokens and the logits fingerprint it produces alone on an idle engine; the engine must go
idle and give back every page."""

from __future__ import annotations

import random
from dataclasses import dataclass, field
from typing import Dict, List, Tuple

from .config.engine import EngineConfig, SamplingParams
from .engine.engine import Engine


@dataclass
class Outcome:
    requests_checked: int = 0
    token_mismatch: int = 0
    fingerprint_mismatch: int = 0
    hangs: int = 0
    leaks: int = 0
    preemptions: int = 0
    prefix_hits: int = 0
    first_bad_trace: int = -1
    notes: List[str] = field(default_factory=list)

    def violations(self) -> int:
        return self.token_mismatch + self.fingerprint_mismatch + self.hangs + self.leaks


class Simulator:
    def __init__(self, model, dtype: str, block_size: int = 16, verbose: bool = False, executor_factory=None):
        self.model, self.dtype, self.block_size, self.verbose = model, dtype, block_size, verbose
        self.vocab = model.assembled.spec.vocab_size if model is not None else 97
        self.max_len = model.assembled.spec.max_positions if model is not None else 1 << 20
        self._refs: Dict[Tuple, Tuple[List[int], int]] = {}
        self._executor_factory = executor_factory

    def _engine(self, cfg: EngineConfig) -> Engine:
        ex = self._executor_factory(cfg) if self._executor_factory else None
        return Engine(self.model, None, cfg, executor=ex)

    def reference(self, prompt: List[int], sp: SamplingParams) -> Tuple[List[int], int]:
        """The request alone: no prefix cache, one step per prompt, just enough pages
        (sim/simulate.cpp:102-118)."""
        key = (tuple(prompt), sp.temperature, sp.seed, sp.max_new_tokens, sp.ignore_eos)
        if key not in self._refs:
            cfg = EngineConfig(num_blocks=(len(prompt) + sp.max_new_tokens) // self.block_size + 2,
                               max_batched_tokens=4096, max_num_seqs=1, prefix_caching=False,
                               block_size=self.block_size, dtype=self.dtype)
            e = self._engine(cfg)
            rid = e.add_request(prompt, sp)
            while not e.idle():
                e.step()
            self._refs[key] = (list(e.result(rid).tokens), e.result(rid).logits_fingerprint)
        return self._refs[key]

    def run_trace(self, seed: int, out: Outcome) -> None:
        rng = random.Random(seed)
        V, bs = self.vocab, self.block_size
        prefixes = [[rng.randrange(4, V) for _ in range(bs * rng.randint(1, 3) if rng.random() < 0.5 else rng.randint(8, 48))]
                    for _ in range(3)]                      # page-aligned prefixes are the edge case
        reqs = []
        max_need = 0
        for i in range(rng.randint(1, 10)):
            if i > 0 and rng.random() < 0.15:
                prompt = list(reqs[rng.randrange(i)][0])    # exact repeat of an earlier prompt
            else:
                prompt = list(rng.choice(prefixes)) if rng.random() < 0.5 else []
                prompt += [rng.randrange(V) for _ in range(rng.randint(0 if prompt else 1, 40))]
            sp = SamplingParams(temperature=0.0 if rng.random() < 0.5 else rng.uniform(0.3, 1.5),
                                seed=rng.getrandbits(63), max_new_tokens=rng.randint(1, 24),
                                ignore_eos=rng.random() < 0.5)
            if len(prompt) + sp.max_new_tokens > self.max_len:
                prompt = prompt[:self.max_len - sp.max_new_tokens]
            arrival = 0 if rng.random() < 0.3 else rng.randint(0, 30)
            cancel = arrival + rng.randint(0, 20) if rng.random() < 0.15 else -1
            reqs.append((prompt, sp, arrival, cancel))
            max_need = max(max_need, len(prompt) + sp.max_new_tokens)
        cfg = EngineConfig(max_batched_tokens=rng.randint(4, 64), max_num_seqs=rng.randint(1, 8),
                           prefix_caching=rng.random() < 0.7, block_size=bs, dtype=self.dtype)
        cfg.num_blocks = (max_need + 1 + bs - 1) // bs + rng.randint(0, 12)
        e = self._engine(cfg)
        ids = [-1] * len(reqs)
        added, hung = 0, True
        for step in range(20000):
            for i, (prompt, sp, arrival, cancel) in enumerate(reqs):
                if arrival == step:
                    ids[i] = e.add_request(prompt, sp)
                    added += 1
                if cancel == step and ids[i] >= 0:
                    e.cancel(ids[i])
            if added == len(reqs) and e.idle():
                hung = False
                break
            e.step()
        if hung:
            out.hangs += 1
            out.notes.append(f"trace {seed}: engine did not finish\n{e.debug_state()}")
            return
        if e.free_blocks != cfg.num_blocks:
            out.leaks += 1
            out.notes.append(f"trace {seed}: {cfg.num_blocks - e.free_blocks} pages not given back")
        out.preemptions += e.stats.preemptions
        out.prefix_hits += e.stats.prefix_hit_tokens
        for i, (prompt, sp, _, _) in enumerate(reqs):
            got = e.result(ids[i])
            if got.cancelled:
                continue
            ref_tokens, ref_print = self.reference(prompt, sp)
            out.requests_checked += 1
            if got.tokens != ref_tokens:
                out.token_mismatch += 1
                out.notes.append(f"trace {seed} request {i}: tokens differ")
            elif got.logits_fingerprint != ref_print:
                out.fingerprint_mismatch += 1
                out.notes.append(f"trace {seed} request {i}: same tokens, different logits")

    def run(self, traces: int, seed: int = 1, only: int = -1) -> Outcome:
        out = Outcome()
        for t in range(traces):
            if only >= 0 and t != only:
                continue
            before = out.violations()
            self.run_trace(seed * 1000003 + t, out)
            if out.violations() > before and out.first_bad_trace < 0:
                out.first_bad_trace = t
        return out

    @staticmethod
    def report(label: str, o: Outcome, traces: int) -> str:
        line = (f"{label:<28s} traces={traces} requests={o.requests_checked} token_mismatch={o.token_mismatch} "
                f"logit_mismatch={o.fingerprint_mismatch} hangs={o.hangs} leaks={o.leaks} | "
                f"preemptions={o.preemptions} prefix_hit_tokens={o.prefix_hits}")
        if o.first_bad_trace >= 0:
            line += f" | first failing trace={o.first_bad_trace}"
        return line
