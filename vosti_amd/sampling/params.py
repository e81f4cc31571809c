"""Sampling parameters and the per-request random stream.

The reference samples greedily only (python/vosti_kernels/kernels.py:1088-1104)
and stops on max_tokens or on one of up to three end tokens unless they are
ignored (src/exec/request_state.rs:97-187, 418-446).  Temperature sampling is
this engine's own: the uniform number that picks output token i of a request is
a function of (the request's seed, i) alone, so what a request generates does
not depend on its companions in a batch or on how its work was cut.
"""
from __future__ import annotations

from dataclasses import dataclass

_MASK = (1 << 64) - 1


@dataclass(frozen=True)
class SamplingParams:
    max_tokens: int = 8              # new tokens to generate (the reference's VOSTI_MAX_TOKENS default)
    temperature: float = 0.0         # 0: greedy
    seed: int = 0
    eos_token_ids: tuple[int, ...] = ()
    ignore_eos: bool = False

    def __post_init__(self):
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if len(self.eos_token_ids) > 3:
            raise ValueError("at most three end tokens")


def _mix64(z: int) -> int:
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def uniform_for(seed: int, output_index: int) -> float:
    """The uniform number in [0, 1) for output token ``output_index`` of a request with ``seed``: 24 bits."""
    z = _mix64((_mix64(seed & _MASK) ^ ((output_index * 0x9E3779B97F4A7C15) & _MASK)) & _MASK)
    return (z >> 40) * 2.0 ** -24
