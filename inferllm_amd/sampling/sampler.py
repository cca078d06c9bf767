"""The device sampler: picks the next token of every sequence of a step."""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..kernels import ops
from .params import SamplingParams


def _as_i64(u: int) -> int:
    return u - (1 << 64) if u >= (1 << 63) else u


class Sampler:
    """Greedy (argmax kernel) or the reference's temperature / top-k / top-p / repeat
    penalty sampler (sample kernel).  A draw depends on the request's seed and on
    how many tokens the request has drawn, not on the rest of the batch."""

    def __init__(self, params: SamplingParams, device):
        params.validate()
        self.params = params
        self.device = device

    def __call__(self, logits: torch.Tensor, seeds: Sequence[int], counters: Sequence[int],
                 histories: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """logits float32 [B, V] on the device -> one token id per row (host list)."""
        p = self.params
        if p.greedy:
            return ops.argmax(logits.contiguous()).tolist()
        B = logits.shape[0]
        last = None
        if p.repeat_penalty != 1.0 and p.repeat_last_n > 0 and histories is not None:
            n = p.repeat_last_n
            rows = [([-1] * n + [int(t) for t in h])[-n:] for h in histories]
            last = torch.tensor(rows, dtype=torch.int32, device=self.device)
        seeds_t = torch.tensor([_as_i64(int(s)) for s in seeds], dtype=torch.int64, device=self.device)
        counters_t = torch.tensor([int(c) for c in counters], dtype=torch.int32, device=self.device)
        return ops.sample(logits.contiguous(), p.temperature, p.top_k, p.top_p, p.repeat_penalty,
                          last, seeds_t, counters_t).tolist()
