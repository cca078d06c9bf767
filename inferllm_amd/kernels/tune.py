"""Measure the dispatch tables of `kernels.plan` for a model's matrix shapes on this GPU.

    python -m inferllm_amd.kernels.tune CONFIG.json [CONFIG.json ...] [--max-rows 8192]

For every config.json it builds one layer of the model with random weights, takes the matrices
the parts really multiply by (fused q|k|v and gate|up included) and times, per shape: from how
few rows the thin matrices go through planes, and for products of many rows the whole product
against its cuts, per class of 256 rows up to --max-rows, and whole against filled up to 256
rows for 65 to 255 rows.  It prints the tables as Python literals, ready for
`FIXED_PLANES_FROM`, `FIXED_CUTS` and `FIXED_ROWS_FROM` (from how few rows the fused q|k|v
product takes the kernel that shares X through LDS).  Entries that say "whole" are left out: that is the rule
for unlisted shapes anyway.
"""
from __future__ import annotations

import argparse
import json
import sys


def matrices(engine):
    """Distinct bfloat16 matrices of the engine's parts, as (shape, `ops.Weight` or tensor)."""
    import torch

    from . import ops
    seen = {}
    for part in engine.model.every_part():
        if part is engine.model.head or part is engine.model.embedding:
            continue                  # float32 logits never go through the products planned
                                      # here, and the embedding table is not multiplied at all
        for w in vars(part).values():
            plain = ops.plain_weight(w) if isinstance(w, (ops.Weight, torch.Tensor)) else None
            if plain is not None and plain.dim() == 2 and plain.dtype == torch.bfloat16:
                seen.setdefault(tuple(plain.shape), w)
    return seen


MARGIN = 0.93       # a table entry must win by 7 %: what is within the clock's noise stays "whole"


def tune_config(cfg: dict, max_rows: int, repeats: int, say, rows_only: bool = False) -> tuple:
    import torch

    from .. import Engine
    from . import ops
    from .plan import NEVER_BELOW, Plan
    one = dict(cfg, num_hidden_layers=1)
    eng = Engine.from_random(one, seed=0, dtype="bfloat16", max_batch=1, max_seq_len=64,
                             decode_copies=True, plan=Plan())
    ops.use_plan(Plan())
    planes, cuts, rows = {}, {}, {}
    for part in eng.model.every_part():
        # a mixer that keeps a fused q|k|v matrix with its head geometry (the attention part)
        w = getattr(part, "w_qkv", None)
        if isinstance(w, ops.Weight) and w.mode == "qkv" and w.tiled is not None and w.shape[1] % 64 == 0:
            key = ("qkv",) + tuple(w.shape)
            if key not in rows:
                votes = sorted(ops.measure_rows_from_qkv(w, part.nh, part.nkv, part.hd)
                               for _ in range(repeats))
                rows[key] = votes[len(votes) // 2]
                say(f"  q|k|v {w.shape[0]} x {w.shape[1]}: shared-X kernel from {rows[key]} rows (runs: {votes})")
        # a feed-forward that keeps a fused gate|up matrix in its fused kernel's tile order
        w = getattr(part, "w_gate_up", None)
        if isinstance(w, ops.Weight) and w.mode == "gate_up" and w.tiled is not None and w.shape[1] % 64 == 0:
            key = ("gate_up",) + tuple(w.shape)
            if key not in rows:
                votes = sorted(ops.measure_rows_from_gate_up(w) for _ in range(repeats))
                rows[key] = votes[len(votes) // 2]
                say(f"  gate|up {w.shape[0]} x {w.shape[1]}: shared-X kernel from {rows[key]} rows (runs: {votes})")
    rows = {k: v for k, v in rows.items() if v != ops.ROWS_FROM}
    if rows_only:
        return planes, cuts, rows
    for (N, K), w in sorted(matrices(eng).items()):
        plain = ops.plain_weight(w)
        if (isinstance(w, ops.Weight) and w.mode == "plain" and w.tiled is not None and K >= 2 * N
                and N <= ops.MID_MAX_COLS and N % 4 == 0):
            votes = sorted(ops.measure_planes_from(w) for _ in range(repeats))
            first = votes[len(votes) // 2]
            say(f"  planes {N} x {K}: from {first} rows (runs: {votes})")
            if first != NEVER_BELOW:
                planes[(N, K)] = first
        for rows32 in range(ops.PAD_MIN_ROWS // 32 + 1, ops.PAD_ROWS // 32 + 1):
            M = min(rows32 * 32, ops.PAD_ROWS - 1)
            x = torch.randn(M, K, device=plain.device).to(torch.bfloat16)
            votes = [ops.measure_plan(x, plain, [(), ("pad", ops.PAD_ROWS)], MARGIN) for _ in range(repeats)]
            best = max(set(votes), key=votes.count)
            if best:
                cuts[("pad", rows32, N, K)] = best
        if N < ops.PLAN_MIN_COLS:
            continue
        for rows256 in range(ops.PLAN_MIN_ROWS // 256, max_rows // 256 + 1):
            M = rows256 * 256
            x = torch.randn(M, K, device=plain.device).to(torch.bfloat16)
            votes = [ops.measure_plan(x, plain, None, MARGIN) for _ in range(repeats)]
            best = max(set(votes), key=votes.count)
            if best:
                cuts[(rows256, N, K)] = best
        say(f"  products {N} x {K}: {sum(1 for k in cuts if k[-2:] == (N, K))} classes are not whole")
    return planes, cuts, rows


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="tune", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("configs", nargs="+", help="config.json files")
    ap.add_argument("--max-rows", type=int, default=8192, help="largest step (rows) to plan for")
    ap.add_argument("--repeats", type=int, default=3, help="measurements per entry; the majority wins")
    ap.add_argument("--rows-only", action="store_true",
                    help="measure FIXED_ROWS_FROM only (the fused q|k|v and gate|up products)")
    args = ap.parse_args(argv)
    say = lambda m: print(m, file=sys.stderr, flush=True)
    planes, cuts, rows = {}, {}, {}
    for path in args.configs:
        with open(path, "r", encoding="utf-8") as f:
            cfg = json.load(f)
        say(f"{path}:")
        p, c, r = tune_config(cfg, args.max_rows, args.repeats, say, args.rows_only)
        planes.update(p)
        cuts.update(c)
        rows.update(r)
    print("FIXED_PLANES_FROM = {")
    for k in sorted(planes):
        print(f"    {k}: {planes[k]},")
    print("}")
    print("FIXED_CUTS = {")
    for k in sorted(cuts, key=repr):
        print(f"    {k}: {cuts[k]},")
    print("}")
    print("FIXED_ROWS_FROM = {")
    for k in sorted(rows):
        print(f"    {k}: {rows[k]},")
    print("}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
