"""Per-request sampling options and the uniform numbers that drive a request's draws.

The options and their meanings are those of the reference's ``sample`` (``sampling.py:141-173``):
``temperature`` 0 is greedy and ignores the rest; otherwise logits are divided by it, ``top_k``
(0: off) keeps the k largest, ``top_p`` (1: off) the smallest set of top tokens whose mass
reaches p.  The reference draws from torch's global generator (``sampling.py:173``), so what it
samples depends on what else is in a batch; here the n-th draw of a request is a pure function
of the request's ``seed`` and n.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

import numpy as np

_MASK = (1 << 64) - 1


@dataclass
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int = 0
    max_new_tokens: int = 16
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError(f"temperature must be >= 0 (got {self.temperature}); 0 means greedy")
        if self.max_new_tokens < 1:
            raise ValueError(f"max_new_tokens must be >= 1 (got {self.max_new_tokens})")
        if self.top_k < 0:
            raise ValueError(f"top_k must be >= 0 (got {self.top_k}); 0 turns it off")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform_for(seed: int, draw_index: int) -> float:
    """The uniform number in [0, 1) of a request's ``draw_index``-th draw (24 bits, exact in float32)."""
    h = _splitmix64(_splitmix64(seed & _MASK) ^ ((draw_index + 1) * 0xD6E8FEB86659FD93 & _MASK))
    return (h >> 40) / float(1 << 24)


def _splitmix64_each(x: np.ndarray) -> np.ndarray:
    x = x + np.uint64(0x9E3779B97F4A7C15)          # unsigned 64-bit arrays wrap around, as the masks above do
    x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
    x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
    return x ^ (x >> np.uint64(31))


def uniforms_for(seeds: Sequence[int], draw_indices: Sequence[int]) -> np.ndarray:
    """``uniform_for`` of each (seed, draw index), as float32: the same numbers, computed for a whole batch at once."""
    seed = np.array([s & _MASK for s in seeds], dtype=np.uint64)
    draw = np.array([(n + 1) & _MASK for n in draw_indices], dtype=np.uint64)
    h = _splitmix64_each(_splitmix64_each(seed) ^ (draw * np.uint64(0xD6E8FEB86659FD93)))
    return ((h >> np.uint64(40)).astype(np.float32)) / np.float32(1 << 24)
