"""Helpers of the replay tests: seeded requests, the four ways of cutting them into steps (whole; most of
it in one step and the last 32 tokens one by one; portions of changing size down to two tokens and one;
mixed with other requests in a pool below their demand), and a driver that runs steps through a Replayer."""

from __future__ import annotations

import random
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch


def requests_for(vocab: int, seed: int, lengths: Sequence[int]) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def all_wanted(rid: str, toks: Sequence[int]) -> dict:
    return {"id": rid, "tokens": list(toks), "want": list(range(len(toks)))}


def whole_steps(rid: str, toks: Sequence[int]) -> List[dict]:
    return [{"entries": [all_wanted(rid, toks)], "end": [rid]}]


def tail_steps(rid: str, toks: Sequence[int], tail: int = 32) -> List[dict]:
    n = len(toks)
    tail = min(tail, n - 1)
    steps = [{"entries": [all_wanted(rid, toks[:n - tail])]}]
    steps += [{"entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}]} for i in range(n - tail, n)]
    steps[-1]["end"] = [rid]
    return steps


def portion_steps(rid: str, toks: Sequence[int], seed: int) -> List[dict]:
    """Portions of changing size: twos and ones among sizes up to 31, a different run for every seed."""
    rng = random.Random(seed)
    steps, pos, n = [], 0, len(toks)
    while pos < n:
        size = min(n - pos, rng.choice([1, 2, 2, 3, 5, 16, 17, 31]))
        steps.append({"entries": [all_wanted(rid, toks[pos:pos + size])]})
        pos += size
    steps[-1]["end"] = [rid]
    return steps


def mixed_steps(reqs: Dict[str, List[int]], seed: int, page: int, max_live: int = 4) -> Tuple[List[dict], int]:
    """All requests in one trace: at most ``max_live`` live at a time, in every step a random subset of the live
    ones, each with a portion of 2 to 40 tokens or, as a decoding request would, a single token; a request may
    sit a step out; one that is through ends and the next one comes in.  Returns the steps and the most
    tokens ever held at once, every request's count rounded up to whole pages (the pool to ask for)."""
    rng = random.Random(seed)
    waiting = list(reqs)
    live: List[str] = []
    done = {rid: 0 for rid in reqs}
    steps: List[dict] = []
    most = 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            live.append(waiting.pop(0))
        chosen = [rid for rid in live if rng.random() < 0.7] or [rng.choice(live)]
        rng.shuffle(chosen)
        entries, end = [], []
        for rid in chosen:
            left = len(reqs[rid]) - done[rid]
            size = min(left, 1 if rng.random() < 0.5 else rng.randint(2, 40))
            entries.append(all_wanted(rid, reqs[rid][done[rid]:done[rid] + size]))
            done[rid] += size
        held = sum((done[rid] + page - 1) // page * page for rid in live)
        most = max(most, held)
        for rid in chosen:
            if done[rid] == len(reqs[rid]):
                end.append(rid)
                live.remove(rid)
        steps.append({"entries": entries, "end": end})
    assert all(done[r] == len(reqs[r]) for r in reqs)
    return steps, most


def run_steps(replayer, steps: Sequence[dict]) -> Dict[str, np.ndarray]:
    """{request: [its wanted rows in order, vocab]}; the manager's invariants are checked after every step."""
    out: Dict[str, list] = {}
    for st in steps:
        lg = replayer.step(st["entries"])
        row = 0
        for e in st["entries"]:
            for _ in e["want"]:
                out.setdefault(e["id"], []).append(lg[row])
                row += 1
        replayer.step([], st.get("end", []))
        replayer.manager.check()
    return {k: np.stack(v) for k, v in out.items()}


# Largest allowed |engine - plain| relative to the largest |logit| of the request.  32-bit: a few units of 2^-24
# per accumulation.  bfloat16: engine and plain model round to bfloat16 at the same places (attention weights
# within the same partitions of keys), so most positions agree to 32-bit accuracy (observed medians: 5e-8 to
# 1e-7); where a value lies so close to the middle between two bfloat16 numbers that the two roundings part, one
# element differs by 2^-9 of its size, which the later layers and, through the cache, the later positions
# inherit (observed maxima: 4e-3 with the tiny configurations' own weights, 1.2e-2 with weights that make
# attention peaked).  So the maximum has a loose bound and, for a model of one layer, where a differing rounding
# stays at its position, the median over positions a tight one: a fault in a formula moves every position.
MAX_TOL = {"float32": 2e-5, "bfloat16": 1e-2}
MEDIAN_TOL = {"float32": 5e-6, "bfloat16": 5e-7}


def check_against_plain(got: np.ndarray, ref: np.ndarray, dtype: str, what: str, max_tol=None, median: bool = False) -> None:
    """Assert the bounds above for the logits [positions, vocab] of one request and print what was observed.
    ``median``: also the bound on the median over positions (32-bit mode, or a model of one layer: with
    more layers one differing rounding reaches most later positions through the cache)."""
    scale = np.abs(ref).max()
    per_row = np.abs(got - ref).max(axis=1) / scale
    bound = MAX_TOL[dtype] if max_tol is None else max_tol
    print(f"{what} {dtype}: max error {per_row.max():.2e} of the largest logit {scale:.3f} (bound {bound:.0e}), "
          f"median over positions {np.median(per_row):.2e} (bound {MEDIAN_TOL[dtype]:.0e}), "
          f"positions within 1e-5: {(per_row <= 1e-5).mean():.2f}")
    assert per_row.max() <= bound, f"{what}: worst at position {int(per_row.argmax())}: {per_row.max():.3e}"
    if median or dtype == "float32":
        assert np.median(per_row) <= MEDIAN_TOL[dtype], f"{what}: median error over positions {np.median(per_row):.3e}"
