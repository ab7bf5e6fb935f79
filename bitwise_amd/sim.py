"""Randomized scheduling scenarios against a solo-run oracle (the role of the reference's simulator,
sim/simulate.cpp:81-217: a request's tokens and logits fingerprint must be those it produces alone on an idle
engine, the engine must go idle, and every page and slot must come back).

What is drawn is this engine's own: the page size, whether decode steps are replayed from graphs and launched
ahead of their tokens, the model length, budgets and pool sizes that force portions and preemption, and workloads
built to hit what those knobs guard: waves of arrivals that double (1, 2, 4, 8 requests: decode steps cross the
graph buckets and a request joins while a step launched ahead is in flight), long leashes that end at an
end-of-sequence token in the middle of such a run, cancellations timed into the decoding phase, prompts that
share prefixes ending on and off a page edge, exact repeats, decode-heavy and prefill-heavy mixes.  The oracle
runs every request alone with one fixed page size, without graphs, run-ahead or prefix cache, so a scenario
also checks that none of the knobs reaches the bits.
"""

from __future__ import annotations

import random
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

from .config.engine import EngineConfig, SamplingParams
from .engine.engine import Engine

ORACLE_PAGE = 16
STEP_GUARD = 20000
KINDS = ("waves", "decode_heavy", "prefill_heavy", "shared_prefixes")


@dataclass
class Arrival:
    prompt: List[int]
    params: SamplingParams
    at_step: int
    cancel_at: int = -1                 # engine step at which the client gives up (-1: never)


@dataclass
class Scenario:
    """One drawn workload and the engine it runs on."""
    seed: int
    kind: str
    engine: EngineConfig
    arrivals: List[Arrival]

    def describe(self) -> str:
        e = self.engine
        return (f"scenario {self.seed} [{self.kind}] {len(self.arrivals)} requests; page {e.block_size}, pool {e.num_blocks}, "
                f"budget {e.max_batched_tokens}, seqs {e.max_num_seqs}, len {e.max_model_len}, graphs {e.use_graphs}, "
                f"ahead {e.run_ahead}, prefix cache {e.prefix_caching}, decode phases {e.decode_phases}, portions to {e.portion_align}")


@dataclass
class Tally:
    scenarios: int = 0
    requests_compared: int = 0
    wrong_tokens: int = 0
    wrong_logits: int = 0
    never_idle: int = 0
    pages_lost: int = 0
    errors: int = 0                     # the engine raised (an injected bug may trip an internal check)
    preemptions: int = 0
    prefix_hit_tokens: int = 0
    ended_by_eos: int = 0
    cancelled: int = 0
    first_failing: int = -1
    knobs_seen: Dict[str, set] = field(default_factory=dict)
    notes: List[str] = field(default_factory=list)

    def violations(self) -> int:
        return self.wrong_tokens + self.wrong_logits + self.never_idle + self.pages_lost + self.errors

    def line(self, label: str) -> str:
        text = (f"{label}: {self.scenarios} scenarios, {self.requests_compared} requests compared with their solo runs; "
                f"wrong tokens {self.wrong_tokens}, same tokens but other logits {self.wrong_logits}, never idle {self.never_idle}, "
                f"pages or slots lost {self.pages_lost}, engine errors {self.errors}; on the way: {self.preemptions} preemptions, "
                f"{self.prefix_hit_tokens} prefix-hit tokens, {self.ended_by_eos} ended by end-of-sequence, {self.cancelled} cancelled")
        if self.first_failing >= 0:
            text += f"; first failing scenario: {self.first_failing}"
        return text


class Simulator:
    """``model`` None with an ``executor_factory`` runs the scenarios on a stand-in device (the scheduler's CPU
    tests); ``fault`` switches one of the engine's test-only bugs on in the scenarios' engines, never in the oracle's."""

    def __init__(self, model, dtype: str, verbose: bool = False, executor_factory: Optional[Callable] = None,
                 fault: int = 0, page_sizes=(8, 16, 32, 64), vocab: Optional[int] = None, max_len: Optional[int] = None):
        self.model, self.dtype, self.verbose, self.fault = model, dtype, verbose, fault
        spec = model.assembled.spec if model is not None else None
        self.vocab = vocab or (spec.vocab_size if spec else 97)
        self.max_len = max_len or (spec.max_positions if spec else 1 << 20)
        self.page_sizes = tuple(page_sizes)
        self._factory = executor_factory
        self._solo: Dict[Tuple, Tuple[List[int], int]] = {}

    # ------------------------------------------------------------------ engines
    def _engine(self, cfg: EngineConfig) -> Engine:
        return Engine(self.model, None, cfg, executor=self._factory(cfg) if self._factory else None)

    def solo(self, prompt: List[int], sp: SamplingParams) -> Tuple[List[int], int]:
        """The request alone on an idle engine: its whole prompt in one step, pages of one fixed size, no prefix
        cache, no graphs, nothing launched ahead, no injected bug."""
        key = (tuple(prompt), sp.temperature, sp.seed, sp.max_new_tokens, sp.ignore_eos)
        if key not in self._solo:
            cfg = EngineConfig(num_blocks=(len(prompt) + sp.max_new_tokens) // ORACLE_PAGE + 2, max_batched_tokens=4096,
                               max_num_seqs=1, prefix_caching=False, block_size=ORACLE_PAGE, dtype=self.dtype,
                               use_graphs=False, run_ahead=False)
            e = self._engine(cfg)
            rid = e.add_request(prompt, sp)
            while not e.idle():
                e.step()
            self._solo[key] = (list(e.result(rid).tokens), e.result(rid).logits_fingerprint)
        return self._solo[key]

    # ------------------------------------------------------------------ drawing a scenario
    def draw(self, seed: int) -> Scenario:
        rng = random.Random(seed)
        kind = KINDS[rng.randrange(len(KINDS))]
        page = rng.choice(self.page_sizes)
        V = self.vocab

        def tokens(n: int) -> List[int]:
            return [rng.randrange(V) for _ in range(n)]

        def sampling(new_tokens: int, leash: bool = False) -> SamplingParams:
            greedy = rng.random() < 0.4
            # a long leash: the request runs until an end-of-sequence token happens to be chosen
            return SamplingParams(temperature=0.0 if greedy else rng.uniform(0.4, 1.4), seed=rng.getrandbits(48),
                                  max_new_tokens=new_tokens, ignore_eos=not leash)

        arrivals: List[Arrival] = []
        if kind == "waves":
            step, size = 0, 1
            for _ in range(rng.randint(2, 4)):              # 1, 2, 4, 8 requests: each wave lands in the decoding of the last
                for _ in range(size):
                    leash = rng.random() < 0.35
                    arrivals.append(Arrival(tokens(rng.randint(1, 12)), sampling(rng.randint(40, 90) if leash else rng.randint(6, 30), leash), step))
                step += rng.randint(2, 9)
                size *= 2
        elif kind == "decode_heavy":
            for _ in range(rng.randint(1, 6)):
                leash = rng.random() < 0.5
                arrivals.append(Arrival(tokens(rng.randint(1, 9)), sampling(rng.randint(30, 80), leash), rng.randint(0, 6)))
        elif kind == "prefill_heavy":
            for _ in range(rng.randint(2, 7)):
                arrivals.append(Arrival(tokens(rng.randint(30, 150)), sampling(rng.randint(1, 4)), rng.randint(0, 12)))
        else:
            # prefixes that end exactly on a page edge, one token before it and one behind it; the same prompt twice
            stems = [tokens(page * rng.randint(1, 3) + rng.choice((-1, 0, 0, 1, rng.randint(2, page)))) for _ in range(rng.randint(1, 3))]
            for i in range(rng.randint(3, 9)):
                if arrivals and rng.random() < 0.2:
                    prompt = list(rng.choice(arrivals).prompt)
                else:
                    # (now and then the stem alone: a prompt that ends on a page edge and is wholly in the cache)
                    prompt = list(rng.choice(stems)) + tokens(0 if rng.random() < 0.3 else rng.randint(1, 30))
                arrivals.append(Arrival(prompt or tokens(1), sampling(rng.randint(1, 20), rng.random() < 0.2), rng.randint(0, 25)))
        for a in arrivals:
            room = self.max_len - a.params.max_new_tokens
            if len(a.prompt) > room:
                a.prompt = a.prompt[:max(1, room)]
                a.params.max_new_tokens = min(a.params.max_new_tokens, self.max_len - len(a.prompt))
            if rng.random() < 0.15:
                # the client gives up somewhere between the arrival and well into the decoding
                a.cancel_at = a.at_step + rng.randint(0, 4 + a.params.max_new_tokens)
        longest = max(len(a.prompt) + a.params.max_new_tokens for a in arrivals)
        seqs = rng.randint(1, 8) if kind != "waves" else rng.choice((2, 4, 8, 16))
        pressure = rng.random()
        need = (longest + 1 + page - 1) // page
        pool = need + (rng.randint(0, 3) if pressure < 0.5 else rng.randint(4, 8 * need))
        budget = rng.randint(2, 24) if rng.random() < 0.5 else rng.randint(25, 256)
        model_len = longest if rng.random() < 0.3 else min(self.max_len, longest + rng.randint(1, 64))
        cfg = EngineConfig(num_blocks=pool, max_batched_tokens=budget, max_num_seqs=seqs, prefix_caching=rng.random() < 0.7,
                           block_size=page, dtype=self.dtype, max_model_len=model_len, use_graphs=rng.random() < 0.7,
                           run_ahead=rng.random() < 0.7, fault=self.fault)
        cfg.decode_phases = rng.random() < 0.3          # (the last draws: the scenarios of a seed are what they were without them)
        cfg.portion_align = rng.choice((1, 4, 16, 64))
        return Scenario(seed, kind, cfg, arrivals)

    # ------------------------------------------------------------------ running one
    def run_scenario(self, sc: Scenario, tally: Tally) -> None:
        tally.scenarios += 1
        for name in ("block_size", "use_graphs", "run_ahead", "prefix_caching", "decode_phases", "portion_align"):
            tally.knobs_seen.setdefault(name, set()).add(getattr(sc.engine, name))
        tally.knobs_seen.setdefault("kind", set()).add(sc.kind)
        try:
            e = self._engine(sc.engine)
            ids: List[int] = [-1] * len(sc.arrivals)
            pending = len(sc.arrivals)
            finished = False
            for step in range(STEP_GUARD):
                for i, a in enumerate(sc.arrivals):
                    if a.at_step == step:
                        ids[i] = e.add_request(a.prompt, a.params)
                        pending -= 1
                    if a.cancel_at == step and ids[i] >= 0:
                        e.cancel(ids[i])
                if pending == 0 and e.idle():
                    finished = True
                    break
                e.step()
        except Exception as err:                            # noqa: BLE001 - whatever an injected bug trips counts as caught
            tally.errors += 1
            tally.notes.append(f"{sc.describe()}\n  the engine raised {type(err).__name__}: {err}")
            return
        if not finished:
            tally.never_idle += 1
            tally.notes.append(f"{sc.describe()}\n  still busy after {STEP_GUARD} steps:\n{e.debug_state()}")
            return
        if not e.manager.all_free():
            tally.pages_lost += 1
            tally.notes.append(f"{sc.describe()}\n  {sc.engine.num_blocks - e.free_blocks} pages were not given back")
        tally.preemptions += e.stats.preemptions
        tally.prefix_hit_tokens += e.stats.prefix_hit_tokens
        for i, a in enumerate(sc.arrivals):
            got = e.result(ids[i])
            if got.cancelled:
                tally.cancelled += 1
                continue
            want_tokens, want_print = self.solo(a.prompt, a.params)
            tally.requests_compared += 1
            tally.ended_by_eos += int(len(got.tokens) < a.params.max_new_tokens)
            if got.tokens != want_tokens:
                tally.wrong_tokens += 1
                first = next((j for j, (x, y) in enumerate(zip(got.tokens, want_tokens)) if x != y), min(len(got.tokens), len(want_tokens)))
                tally.notes.append(f"{sc.describe()}\n  request {i}: token {first} of {len(want_tokens)} is not the solo run's")
            elif got.logits_fingerprint != want_print:
                tally.wrong_logits += 1
                tally.notes.append(f"{sc.describe()}\n  request {i}: the solo run's tokens from other logits")

    def run(self, scenarios: int, seed: int = 1, only: int = -1) -> Tally:
        tally = Tally()
        for t in range(scenarios):
            if only >= 0 and t != only:
                continue
            before = tally.violations()
            self.run_scenario(self.draw(seed * 7919 + t), tally)
            if tally.violations() > before and tally.first_failing < 0:
                tally.first_failing = t
        return tally
