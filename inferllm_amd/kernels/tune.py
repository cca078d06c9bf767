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
    """Distinct bfloat16 matrices that the engine's parts list as having several ways
    (`Part.tunables`), as (shape, `ops.Weight` or tensor)."""
    import torch

    from . import ops
    seen = {}
    for part in engine.model.every_part():
        for _kind, w, _geometry in part.tunables():
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
    plan = Plan()
    eng = Engine.from_random(one, seed=0, dtype="bfloat16", max_batch=1, max_seq_len=64,
                             decode_copies=True, plan=plan)
    ops.use_plan(plan)
    rules = plan.rules
    cuts = {}
    # what the parts themselves list: the thin matrices' planes and the fused products' rows
    for part in eng.model.every_part():
        for kind, w, geometry in part.tunables():
            if rows_only and kind == "plain":
                continue
            entry = ops.tune_product(plan, kind, w, votes=repeats, **geometry)
            if entry is not None:
                say(f"  {entry[0]} {entry[1]}: {entry[2]}")
    planes = {k: v for k, v in plan.planes_from.items() if v != NEVER_BELOW}
    rows = {k: v for k, v in plan.rows_from.items() if v != rules.rows_from}
    if rows_only:
        return planes, cuts, rows
    for (N, K), w in sorted(matrices(eng).items()):
        plain = ops.plain_weight(w)
        for rows32 in range(rules.pad_rows_above // 32 + 1, rules.pad_rows_to // 32 + 1):
            M = min(rows32 * 32, rules.pad_rows_to - 1)
            x = torch.randn(M, K, device=plain.device).to(torch.bfloat16)
            votes = [ops.measure_plan(x, plain, [(), ("pad", rules.pad_rows_to)], MARGIN) for _ in range(repeats)]
            best = max(set(votes), key=votes.count)
            if best:
                cuts[("pad", rows32, N, K)] = best
        if N < rules.cut_min_cols:
            continue
        for rows256 in range(rules.cut_min_rows // 256, max_rows // 256 + 1):
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
