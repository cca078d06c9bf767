"""Per-kernel timing of the engine's own ops with HIP events.

`with kernel_timing() as t: ...; print(t.table())` wraps every function of
`kernels.ops` that launches work, records an event pair around each call and
reports calls, total and mean time per op.  Steps must run eagerly while timing
(`Engine(..., use_graphs=False)`): a captured graph replays without passing through
Python.  The reference has the same switch at build time: `ENABLE_PROFILE` prints
the time of every op (src/core/graph.cpp:21-32).
"""
from __future__ import annotations

import contextlib
from collections import OrderedDict
from typing import Dict, List, Tuple

import torch

from . import ops

_TIMED = ("embed", "add_rmsnorm", "silu_mul", "rope_store", "qkv_rope_store", "gate_up_silu",
          "linear", "linear_add", "linear_planes", "attn_prefill", "attn_decode", "argmax", "sample")


class KernelTimes:
    def __init__(self):
        self.events: Dict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]] = OrderedDict()

    def add(self, name, start, end):
        self.events.setdefault(name, []).append((start, end))

    def totals(self) -> Dict[str, Tuple[int, float]]:
        """op -> (calls, total milliseconds); synchronizes the device."""
        torch.cuda.synchronize()
        return {n: (len(ev), sum(a.elapsed_time(b) for a, b in ev)) for n, ev in self.events.items()}

    def table(self) -> str:
        tot = self.totals()
        whole = sum(ms for _, ms in tot.values()) or 1.0
        lines = [f"{'op':16s} {'calls':>7s} {'total ms':>10s} {'mean us':>9s} {'share':>6s}"]
        for n, (calls, ms) in sorted(tot.items(), key=lambda kv: -kv[1][1]):
            lines.append(f"{n:16s} {calls:7d} {ms:10.3f} {ms / calls * 1e3:9.1f} {100 * ms / whole:5.1f}%")
        return "\n".join(lines)


@contextlib.contextmanager
def kernel_timing():
    times = KernelTimes()
    saved = {}

    depth = [0]                              # ops that call other ops are timed as the outer one

    def wrap(name, fn):
        def timed(*a, **kw):
            if depth[0] or torch.cuda.is_current_stream_capturing():
                return fn(*a, **kw)
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            depth[0] += 1
            try:
                s.record()
                out = fn(*a, **kw)
                e.record()
            finally:
                depth[0] -= 1
            times.add(name, s, e)
            return out
        return timed

    for name in _TIMED:
        saved[name] = getattr(ops, name)
    try:
        for name in _TIMED:
            setattr(ops, name, wrap(name, saved[name]))
        yield times
    finally:
        for name, fn in saved.items():
            setattr(ops, name, fn)
