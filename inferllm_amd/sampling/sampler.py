"""The device sampler: picks the next token of every sequence of a step."""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
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
        self._stage: Optional[torch.Tensor] = None     # pinned [seeds (2 words each) | counters | windows]

    def _upload(self, seeds, counters, windows):
        """One pinned buffer, one copy: (seeds int64 [B], counters int32 [B], windows int32 [B, n] or None)."""
        B = len(seeds)
        n = len(windows[0]) if windows else 0
        words = B * (3 + n)
        if self._stage is None or self._stage.numel() < words:
            self._stage = torch.empty(max(words, 1024), dtype=torch.int32,
                                      pin_memory=torch.device(self.device).type == "cuda")
        host = self._stage[:words]
        flat = host.numpy()                              # shares the pinned memory
        flat[:2 * B].view(np.int64)[:] = [_as_i64(int(s)) for s in seeds]
        flat[2 * B:3 * B] = counters
        if n:
            flat[3 * B:].reshape(B, n)[:] = windows
        dev = host.to(self.device, non_blocking=True)
        return (dev[:2 * B].view(torch.int64), dev[2 * B:3 * B],
                dev[3 * B:].view(B, n) if n else None)

    def __call__(self, logits: torch.Tensor, seeds: Sequence[int], counters: Sequence[int],
                 histories: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """logits float32 [B, V] on the device -> one token id per row (host list)."""
        p = self.params
        if p.greedy:
            return ops.argmax(logits.contiguous()).tolist()
        rows = None
        if p.repeat_penalty != 1.0 and p.repeat_last_n > 0 and histories is not None:
            n = p.repeat_last_n
            rows = [[-1] * (n - min(n, len(h))) + list(h[-n:]) for h in histories]
        seeds_t, counters_t, last = self._upload(seeds, counters, rows)
        return ops.sample(logits.contiguous(), p.temperature, p.top_k, p.top_p, p.repeat_penalty,
                          last, seeds_t, counters_t).tolist()
