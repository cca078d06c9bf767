"""The device sampler: picks the next token of every sequence of a step."""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from .params import SamplingParams


def _as_i64(u: int) -> int:
    return u - (1 << 64) if u >= (1 << 63) else u


class Draw:
    """The tokens of one sampling call: on the device at once (`device`, int32 [B]; `pick(rows)`
    for some of them), on the host when asked for (`tokens()` waits for the copy that was started
    with the draw)."""

    def __init__(self, device_tokens: torch.Tensor, host: torch.Tensor, copied):
        self.device, self._host, self._copied = device_tokens, host, copied

    def pick(self, rows: Sequence[int]) -> torch.Tensor:
        index = torch.tensor(list(rows), dtype=torch.long, device=self.device.device)
        return self.device.index_select(0, index)

    def tokens(self) -> List[int]:
        if self._copied is not None:
            self._copied.synchronize()
        return self._host.tolist()


class Sampler:
    """Greedy (argmax kernel) or the reference's temperature / top-k / top-p / repeat
    penalty sampler (sample kernel).  A draw depends on the request's seed and on
    how many tokens the request has drawn, not on the rest of the batch."""

    def __init__(self, params: SamplingParams, device):
        params.validate()
        self.params = params
        self.device = device
        # pinned [seeds (2 words each) | counters | windows], four in turn: a draw's numbers may
        # still wait for their copy when the next draw's are written
        self._stages: List[Optional[torch.Tensor]] = [None] * 4
        self._back: List[torch.Tensor] = []            # pinned buffers the drawn tokens come back in
        self._turn = 0

    def _upload(self, seeds, counters, windows):
        """One pinned buffer, one copy: (seeds int64 [B], counters int32 [B], windows int32 [B, n] or None)."""
        B = len(seeds)
        n = len(windows[0]) if windows else 0
        words = B * (3 + n)
        stage = self._stages[self._turn]
        if stage is None or stage.numel() < words:
            stage = self._stages[self._turn] = torch.empty(
                max(words, 1024), dtype=torch.int32,
                pin_memory=torch.device(self.device).type == "cuda")
        host = stage[:words]
        flat = host.numpy()                              # shares the pinned memory
        flat[:2 * B].view(np.int64)[:] = [_as_i64(int(s)) for s in seeds]
        flat[2 * B:3 * B] = counters
        if n:
            flat[3 * B:].reshape(B, n)[:] = windows
        dev = host.to(self.device, non_blocking=True)
        return (dev[:2 * B].view(torch.int64), dev[2 * B:3 * B],
                dev[3 * B:].view(B, n) if n else None)

    def needs_histories(self) -> bool:
        """Whether a draw depends on the tokens before it (the repeat penalty's window)."""
        p = self.params
        return (not p.greedy) and p.repeat_penalty != 1.0 and p.repeat_last_n > 0

    def draw(self, logits: torch.Tensor, seeds: Sequence[int], counters: Sequence[int],
             histories: Optional[Sequence[Sequence[int]]] = None,
             latest: Optional[torch.Tensor] = None) -> Draw:
        """logits float32 [B, V] on the device -> one token id per row, chosen on the device; the
        copy to the host is under way when this returns.  At most four draws may be unread.

        `latest` (int32 [B] on the device): every sequence's newest token when the host has not
        read it yet; `histories` then hold the tokens before it, and the repeat penalty's window
        is completed on the device."""
        p = self.params
        self._turn = (self._turn + 1) % 4
        if p.greedy:
            dev = ops.argmax(logits.contiguous())
        else:
            rows = None
            if self.needs_histories() and histories is not None:
                n = p.repeat_last_n
                if latest is None:
                    rows = [[-1] * (n - min(n, len(h))) + list(h[-n:]) for h in histories]
                else:
                    m = n - 1
                    rows = [[-1] * (m - min(m, len(h))) + (list(h[-m:]) if m else []) + [-1]
                            for h in histories]
            seeds_t, counters_t, last = self._upload(seeds, counters, rows)
            if last is not None and latest is not None:
                last[:, -1].copy_(latest)
            dev = ops.sample(logits.contiguous(), p.temperature, p.top_k, p.top_p,
                             p.repeat_penalty, last, seeds_t, counters_t)
        B = dev.numel()
        if not dev.is_cuda:                  # stand-in kernels on the CPU (tests): nothing to wait for
            return Draw(dev, dev, None)
        while len(self._back) < 4:
            self._back.append(torch.empty(1024, dtype=torch.int32, pin_memory=True))
        if self._back[self._turn].numel() < B:
            self._back[self._turn] = torch.empty(B, dtype=torch.int32, pin_memory=True)
        host = self._back[self._turn][:B]
        host.copy_(dev, non_blocking=True)
        copied = torch.cuda.Event()
        copied.record()
        return Draw(dev, host, copied)

    def __call__(self, logits: torch.Tensor, seeds: Sequence[int], counters: Sequence[int],
                 histories: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """logits float32 [B, V] on the device -> one token id per row (host list)."""
        return self.draw(logits, seeds, counters, histories).tokens()
