"""Per-request sampling options and the counter-based random numbers behind them."""

import os
from dataclasses import dataclass
from typing import Optional

_MASK = (1 << 64) - 1


@dataclass(frozen=True)
class SamplingParams:
    """``temperature == 0`` is greedy (the reference's only mode,
    src/scheduler/orca_scheduler.py:250); otherwise tokens are drawn from
    ``softmax(logits / temperature)``.  With a ``seed`` the draws of a request are a
    function of (seed, request id, index of the generated token) only, so they do not
    depend on what else was batched with it."""

    temperature: float = 0.0
    seed: Optional[int] = None
    max_new_tokens: int = 16
    ignore_eos: bool = False

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature cannot be negative")
        if self.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")


def _splitmix64(value: int) -> int:
    value = (value + 0x9E3779B97F4A7C15) & _MASK
    value = ((value ^ (value >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    value = ((value ^ (value >> 27)) * 0x94D049BB133111EB) & _MASK
    return value ^ (value >> 31)


def uniform_for(seed: int, request_key: int, index: int) -> float:
    """A uniform number in [0, 1) with 24 random bits (exact in float32) for draw
    ``index`` of request ``request_key`` under ``seed``."""
    state = _splitmix64(seed & _MASK)
    state = _splitmix64(state ^ (request_key & _MASK))
    state = _splitmix64(state ^ (index & _MASK))
    return (state >> 40) / float(1 << 24)


def fresh_seed() -> int:
    return int.from_bytes(os.urandom(8), "little")
