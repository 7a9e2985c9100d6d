"""Sampling parameters and the random draw.

The reference samples with (temperature, topk, topp) per request
(include/infinicore_infer/models/jiuge.h:85-88) and one uniform draw per request
and step from a host generator that is re-seeded from the machine's entropy each
step (src/models/jiuge/jiuge.cpp:279-284), so its runs cannot be repeated.
Defaults are the reference's: temperature 1.0, topk 1, topp 1.0
(scripts/jiuge.py:539), i.e. greedy.  Here the draw is a pure function of
(seed, request id, number of tokens generated so far): runs repeat, and a
request that is recomputed after losing its pages draws the same numbers.
"""
import hashlib
from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 1.0
    topk: int = 1
    topp: float = 1.0
    seed: int = 0

    def __post_init__(self):
        if not (self.temperature >= 0) or self.temperature == float("inf"):
            raise ValueError("temperature must be a finite number >= 0, got %r" % (self.temperature,))
        if int(self.topk) != self.topk or self.topk < 0:
            raise ValueError("topk must be an integer >= 0 (0 keeps every token), got %r" % (self.topk,))
        if not (0.0 <= self.topp <= 1.0):
            raise ValueError("topp must lie in [0, 1], got %r" % (self.topp,))

    @property
    def greedy(self) -> bool:
        """jiuge.h:85-88: temperature 0 or topk 1 means argmax."""
        return self.temperature == 0 or self.topk == 1


def uniform_draw(seed: int, request_id, step: int) -> float:
    """A number in [0, 1) fixed by (seed, request id, step)."""
    h = hashlib.blake2b(("%d/%s/%d" % (seed, request_id, step)).encode(), digest_size=8).digest()
    return (int.from_bytes(h, "little") >> 11) / float(1 << 53)
