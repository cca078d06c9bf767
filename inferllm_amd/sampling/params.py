"""Sampling options, with the reference's names and meanings (application/chat.cpp:20-39,
src/utils.cpp:31-115), and the stream of uniform numbers the draws use."""
from __future__ import annotations

from dataclasses import dataclass

_M64 = (1 << 64) - 1


@dataclass
class SamplingParams:
    """temperature 0 is greedy (largest logit, lowest id on ties); the reference has
    no greedy branch and divides by its `temp`.  top_k <= 0 and top_p >= 1 switch
    those filters off, repeat_penalty 1 switches the penalty off."""
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    repeat_penalty: float = 1.0
    repeat_last_n: int = 64
    seed: int = 0

    def validate(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
        if not (0 < self.top_p <= 1.0):
            raise ValueError("top_p must be in (0, 1]")
        if self.repeat_penalty <= 0:
            raise ValueError("repeat_penalty must be positive")
        if not (0 <= self.repeat_last_n <= 256):
            raise ValueError("repeat_last_n must be within 0..256")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0


def splitmix64(z: int) -> int:
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def request_seed(seed: int, request_index: int) -> int:
    """The seed of one request's stream: a hash of the call's seed and the request's index."""
    return splitmix64((seed & _M64) * 0x9E3779B97F4A7C15 + request_index + 1)


def uniform(request_seed_: int, counter: int) -> float:
    """The uniform number in [0, 1) of draw `counter` of a request: the same formula
    as `uniform_from` in csrc/sampling.hip (24 bits of a splitmix64 hash)."""
    z = splitmix64((request_seed_ + 0x9E3779B97F4A7C15 * (counter + 1)) & _M64)
    return (z >> 40) / 16777216.0
