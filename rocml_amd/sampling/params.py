"""Sampling parameters and the host-side random number generator.

Fields and defaults are the reference's (rocml/src/sample.rs:17-51): a
temperature of zero or less selects greedy decoding and every other field is
then ignored; ``top_k`` and ``top_p`` are optional; the repeat penalty looks at
the last ``repeat_penalty_window`` tokens of the history.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

_MASK64 = (1 << 64) - 1


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: Optional[int] = None
    top_p: Optional[float] = None
    seed: int = 0
    repeat_penalty: Optional[float] = None
    repeat_penalty_window: int = 64

    @staticmethod
    def greedy() -> "SamplingParams":
        return SamplingParams()

    def is_greedy(self) -> bool:
        return self.temperature <= 0.0

    def penalty_active(self) -> bool:
        """A penalty of 1, or one that is not positive, changes nothing
        (rocml/src/sample.rs:188-191)."""
        p = self.repeat_penalty
        return p is not None and p > 0.0 and abs(p - 1.0) >= 1.1920929e-07


class Rng:
    """xorshift64* (rocml/src/sample.rs:56-83): shifts 12/25/27, multiplier
    ``0x2545F4914F6CDD1D``; a zero seed is replaced by ``0x9E3779B97F4A7C15``;
    a draw is the top 24 bits of the output divided by 2^24."""

    def __init__(self, seed: int):
        seed &= _MASK64
        self.state = seed if seed != 0 else 0x9E3779B97F4A7C15

    def next_u64(self) -> int:
        x = self.state
        x ^= x >> 12
        x ^= (x << 25) & _MASK64
        x ^= x >> 27
        self.state = x
        return (x * 0x2545F4914F6CDD1D) & _MASK64

    def next_f32(self) -> float:
        return float(self.next_u64() >> 40) / float(1 << 24)


def sequence_seed(seed: int, index: int) -> int:
    """Seed of the ``index``-th sequence of a call: each sequence draws from a
    stream of its own so that batching does not change its draws.  The first
    sequence keeps the call's seed, as the reference's single sequence does
    (rocml/src/generate/resumed.rs:175)."""
    if index == 0:
        return seed & _MASK64
    # splitmix64 step over (seed, index): cheap and well spread.
    z = (seed + index * 0x9E3779B97F4A7C15) & _MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
    return z ^ (z >> 31)
