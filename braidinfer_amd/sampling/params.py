"""Sampling options with the reference's names, meanings and defaults
(crates/braidinfer-runtime/src/sampling.rs:7-47), and the uniform numbers the sampler
draws.  The reference seeds a `StdRng` (:188-191); its stream cannot be reproduced
outside Rust, so the generator here is this library's own: a counter-based hash of
(seed, sequence, draw), which gives a sequence the same numbers alone or in any batch.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

_MASK = (1 << 64) - 1


@dataclass
class SamplingParams:
    temperature: float = 1.0            # 0.0: argmax
    top_k: int = 50                     # 0: off
    top_p: float = 1.0                  # 1.0: off
    repetition_penalty: float = 1.0     # 1.0: off; applied once per occurrence in the history
    seed: Optional[int] = None          # None: from the system's entropy
    min_p: float = 0.0                  # 0.0: off; drops tokens with p < min_p * p_max
    logit_bias: Optional[List[Tuple[int, float]]] = None   # (token, delta), added first

    @classmethod
    def greedy(cls) -> "SamplingParams":
        return cls(temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0, seed=None, min_p=0.0,
                   logit_bias=None)

    def validate(self) -> None:
        if self.temperature < 0:
            raise ValueError(f"temperature must be >= 0, got {self.temperature}")
        if self.top_k < 0:
            raise ValueError(f"top_k must be >= 0, got {self.top_k}")
        if not 0 < self.top_p <= 1:
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")
        if not 0 <= self.min_p <= 1:
            raise ValueError(f"min_p must be in [0, 1], got {self.min_p}")
        if self.repetition_penalty <= 0:
            raise ValueError(f"repetition_penalty must be positive, got {self.repetition_penalty}")

    @property
    def is_plain_greedy(self) -> bool:
        return self.temperature == 0.0 and not self.logit_bias and self.repetition_penalty == 1.0


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform_key(seed: int, sequence: int) -> int:
    """What a request's uniform numbers are made from: 64 bits of its seed and its number."""
    h = _splitmix64(seed & _MASK)
    return _splitmix64(h ^ ((sequence * 0xD6E8FEB86659FD93) & _MASK))


def uniform(seed: int, sequence: int, draw: int) -> float:
    """A float in [0, 1) with 24 random bits, a pure function of its arguments (the draw
    kernel of csrc/sampling.hip makes the same from `uniform_key` and the draw's number)."""
    h = _splitmix64(uniform_key(seed, sequence) ^ ((draw * 0xCA5A826395121157) & _MASK))
    return (h >> 40) / float(1 << 24)


def resolve_seed(seed: Optional[int]) -> int:
    return int.from_bytes(os.urandom(8), "little") if seed is None else int(seed)
