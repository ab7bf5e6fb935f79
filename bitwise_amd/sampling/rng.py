"""Counter-based randomness: a uniform in [0, 1) that is a pure function of
(seed, position, stream) (src/engine.cpp:12-16, :35-38).  Sampling never draws from engine
state, so preemption and recomputation cannot shift a request's random numbers."""

from __future__ import annotations

_M64 = (1 << 64) - 1
STREAM_SAMPLE = 0          # streams 1-3 belong to speculative decoding in the reference (src/engine.cpp:31)
FINGERPRINT_BASIS = 1469598103934665603     # start of every request's logits fingerprint (src/engine.h:68)


def mix64(z: int) -> int:
    """The splitmix64 finaliser."""
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def counter_uniform(seed: int, position: int, stream: int = STREAM_SAMPLE) -> float:
    """(z >> 11) * 2**-53, z = mix64(mix64(seed ^ 0x6A09E667F3BCC909) ^ mix64(position*4 + stream))."""
    z = mix64(mix64((seed ^ 0x6A09E667F3BCC909) & _M64) ^ mix64((position * 4 + stream) & _M64))
    return (z >> 11) * 2.0 ** -53
