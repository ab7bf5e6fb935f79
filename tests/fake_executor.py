"""A stand-in for the device in scheduler tests: a 'model' whose next token is a hash of the
whole token sequence as read back from paged storage through the block tables.  If the
scheduler or cache manager ever shares, reuses or loses a page wrongly, the sequence read
back differs from the request's own tokens and the generated tokens change."""

from __future__ import annotations

from typing import Dict, List

from bitwise_amd.cache.manager import GroupSpec

_M64 = (1 << 64) - 1


def _mix(z: int) -> int:
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


AHEAD_TOKEN = -2


class _LazyStep:
    """A launched step of the stand-in device: evaluated when its result is asked for, which the engine does
    in launch order, so reads and writes of the pages happen in the order a device stream would give them."""

    def __init__(self, ex, segments, draw, prints, after):
        self.ex, self.segments, self.draw, self.prints, self.after = ex, segments, draw, prints, after
        self.n = len(draw[0])
        self.decode_rows = len(segments) if all(len(s.tokens) == 1 and tuple(s.want) == (0,) for s in segments) else 0
        self._r = None

    def result(self):
        if self._r is None:
            segs = self.segments
            prev = self.prints
            if self.after is not None:
                toks, prev_prints = self.after.result()
                assert len(toks) == len(segs)
                segs = [type(s)([toks[i]] if s.tokens[0] == AHEAD_TOKEN else s.tokens, s.pos0, s.tables, s.slot, s.want)
                        for i, s in enumerate(segs)]
                prev = prev_prints if prev_prints else None
            assert all(t >= 0 for s in segs for t in s.tokens), "a step ahead of its tokens without the step before"
            logits = self.ex.run(segs)
            tokens = self.ex.sample(logits, *self.draw) if self.n else []
            self._r = (tokens, self.ex.fingerprints(logits, prev) if prev is not None and self.n else [])
        return self._r


class FakeExecutor:
    def __init__(self, page_size: int, vocab_size: int = 97, eos_token_id: int = 3, max_model_len: int = 1 << 20,
                 run_ahead: bool = False):
        self.group_specs = [GroupSpec()]
        self.has_state = False
        self.vocab_size = vocab_size
        self.eos_token_id = eos_token_id
        self.max_model_len = max_model_len
        self.page_size = page_size
        self.pages: Dict[int, List[int]] = {}
        self.steps = 0
        self.rows_run = 0
        self.reset_slots: List[int] = []
        self.steps_ahead = 0
        if run_ahead:        # the device's two-part face: launch now, read back later; a step may be launched ahead
            self.launch = self._launch
            self.can_run_ahead = lambda pend, rows: pend.decode_rows == rows and pend.n == rows

    def reset_slot(self, slot: int) -> None:
        self.reset_slots.append(slot)

    def _launch(self, segments, draw, prints, after=None):
        if after is not None:
            self.steps_ahead += 1
        return _LazyStep(self, segments, draw, prints, after)

    def run(self, segments):
        self.steps += 1
        ps = self.page_size
        for s in segments:                       # every row's token goes into its page slot first
            for i, t in enumerate(s.tokens):
                pos = s.pos0 + i
                page = s.tables[0][pos // ps]
                assert page >= 0
                self.pages.setdefault(page, [None] * ps)[pos % ps] = t
                self.rows_run += 1
        out = []
        for s in segments:
            for w in s.want:
                pos = s.pos0 + w
                h = 1469598103934665603
                for p in range(pos + 1):
                    t = self.pages[s.tables[0][p // ps]][p % ps]
                    assert t is not None, "read of a slot that was never written"
                    h = _mix(h ^ (t + 1))
                out.append(h)
        return out

    def sample(self, logits, temperatures, seeds, positions):
        toks = []
        for h, t, seed, pos in zip(logits, temperatures, seeds, positions):
            if t > 0:
                h = _mix(h ^ _mix(seed * 1000003 + pos))
            toks.append(h % self.vocab_size)
        return toks

    def fingerprints(self, logits, previous):
        return [_mix(p ^ h) for h, p in zip(logits, previous)]
