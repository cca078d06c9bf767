"""Which of several equivalent ways a bfloat16 product takes, as data.

Some products can run in more than one way that differ in speed by shape and in rounding
only: the down projection of few rows through the residual-adding kernel or through planes
(`ops.linear_planes`), a product of many rows whole, cut along its output columns, in two
halves of its rows or filled up to 256 rows.  Which way is taken must not depend on a
stopwatch, or the same request could give other bfloat16 logits in another process.  So
the choice is a table by shape:

* `Plan.fixed()` (what an engine uses unless told otherwise): the tables below, measured once
  on an MI355X for the matrix shapes of LLaMA-2-7B, LLaMA-2-13B, LLaMA-3-8B and LLaMA-2-70B
  (`python -m inferllm_amd.kernels.tune`: the majority of three measurements, and a way other
  than the rule's must win by 7 %), and for every other shape one rule: planes from 17 rows on,
  products of many rows whole.  Nothing is ever timed.
  The third table says from how few rows (below 17) the q|k|v product goes to the kernel that
  shares X through LDS (csrc/gemm_rows.hip) rather than to the few-rows kernel; gate|up and the
  head measured equal or worse there below 17 rows and have no entries.
* `Plan(measure=True)` (`Engine(tune=True)`): a shape that the tables lack is timed the first
  time it is used outside graph capture and the winner is kept; `to_dict()` gives the result,
  which `Engine(plan=...)` pins in another process.

The float32 path has one way per product and no plan.
"""
from __future__ import annotations

from dataclasses import asdict, dataclass
from typing import Dict, Optional, Tuple

NEVER_BELOW = 17          # planes are not taken below 17 rows (the rule for unlisted shapes)


@dataclass
class Rules:
    """What a shape that the tables lack gets, and the ranges of shapes in which a way is a
    candidate at all.  Measured on an MI355X at the LLaMA-2-7B, 13B, 70B and LLaMA-3-8B matrix
    shapes; a plan for other hardware or other shapes carries other numbers, the code none."""
    rows_from: int = 17            # rows from which the products that share X through LDS are taken
                                   # (up to 16 rows the few-rows kernels are the other way)
    planes_most_cols: int = 8192   # output columns up to which planes were measured to pay: product
                                   # and the norm that adds the planes take 0.6 to 0.75 of the vendor
                                   # GEMM's and the norm's time when K >= 2 N, 0.8 to 0.95 when K = N
    planes_min_elements: int = 1 << 22   # smaller matrices are not timed (both ways take a few
                                         # microseconds and the clock would decide)
    pad_rows_above: int = 64       # products of more rows than this and fewer than `pad_rows_to` may be
    pad_rows_to: int = 256         # filled up to `pad_rows_to` rows (4096 x 11008: 60, 82 and 51 us at
                                   # 128, 192 and 256 rows)
    cut_min_rows: int = 1024       # below these no cut of a many-row product ever paid
    cut_min_cols: int = 8192

# (N, K) of a matrix with K >= 2 N -> fewest rows (1, 5, 9, 13 or 17) from which the planes and
# the norm that adds them take less time than the residual-adding few-rows product.
FIXED_PLANES_FROM: Dict[Tuple[int, int], int] = {
    (4096, 11008): 13,
    (4096, 14336): 9,
    (5120, 13824): 1,
    (8192, 28672): 5,
}

# (rows / 256 rounded up, N, K) -> plan of a product of at least 1024 rows and 8192 columns:
# () whole, (c,) cut of the output columns at c, ("rows", n) the rows in n equal parts.
# ("pad", rows / 32 rounded up, N, K) -> () or ("pad", 256) for products of 65 to 255 rows.
FIXED_CUTS: Dict[tuple, tuple] = {
    ('pad', 4, 4096, 11008): ('pad', 256),
    ('pad', 4, 4096, 14336): ('pad', 256),
    ('pad', 5, 4096, 11008): ('pad', 256),
    ('pad', 5, 4096, 14336): ('pad', 256),
    ('pad', 6, 4096, 11008): ('pad', 256),
    ('pad', 6, 4096, 14336): ('pad', 256),
    (10, 27648, 5120): (12288,),
    (11, 22016, 4096): (12288,),
    (11, 27648, 5120): (12288,),
    (11, 8192, 8192): (4096,),
    (12, 22016, 4096): (8192,),
    (12, 27648, 5120): (8192,),
    (12, 57344, 8192): (8192,),
    (13, 15360, 5120): (7680,),
    (13, 22016, 4096): (8192,),
    (13, 28672, 4096): (12288,),
    (13, 8192, 28672): (4096,),
    (14, 10240, 8192): (4096,),
    (14, 15360, 5120): (7680,),
    (14, 22016, 4096): (8192,),
    (14, 28672, 4096): (8192,),
    (15, 10240, 8192): (4096,),
    (15, 22016, 4096): (11008,),
    (15, 27648, 5120): (24576,),
    (15, 8192, 28672): (4096,),
    (16, 10240, 8192): (4096,),
    (16, 22016, 4096): (8192,),
    (16, 27648, 5120): (12288,),
    (17, 10240, 8192): (4096,),
    (17, 12288, 4096): (6144,),
    (17, 22016, 4096): (16384,),
    (17, 8192, 8192): (4096,),
    (18, 15360, 5120): (7680,),
    (18, 22016, 4096): (8192,),
    (19, 10240, 8192): (4096,),
    (19, 8192, 8192): (4096,),
    (20, 10240, 8192): (4096,),
    (20, 22016, 4096): (11008,),
    (20, 28672, 4096): (12288,),
    (20, 8192, 28672): (4096,),
    (20, 8192, 8192): (4096,),
    (21, 10240, 8192): (4096,),
    (21, 22016, 4096): (20480,),
    (21, 27648, 5120): (12288,),
    (21, 28672, 4096): (8192,),
    (22, 15360, 5120): (7680,),
    (23, 8192, 8192): (4096,),
    (24, 12288, 4096): (6144,),
    (24, 22016, 4096): (20480,),
    (24, 28672, 4096): (8192,),
    (25, 22016, 4096): (20480,),
    (25, 27648, 5120): (12288,),
    (25, 28672, 4096): (8192,),
    (26, 10240, 8192): (4096,),
    (26, 27648, 5120): (8192,),
    (27, 10240, 8192): (4096,),
    (27, 12288, 4096): (6144,),
    (27, 15360, 5120): (8192,),
    (27, 22016, 4096): (8192,),
    (28, 10240, 8192): (4096,),
    (28, 22016, 4096): (8192,),
    (28, 8192, 28672): ('rows', 2),
    (29, 15360, 5120): (12288,),
    (29, 28672, 4096): (12288,),
    (30, 15360, 5120): (7680,),
    (30, 22016, 4096): (12288,),
    (31, 15360, 5120): (8192,),
    (31, 22016, 4096): (20480,),
    (32, 22016, 4096): (20480,),
    (32, 27648, 5120): (12288,),
    (4, 27648, 5120): (12288,),
    (5, 28672, 4096): (24576,),
    (6, 22016, 4096): (20480,),
    (6, 27648, 5120): (8192,),
    (7, 10240, 8192): (8192,),
    (7, 22016, 4096): (8192,),
    (7, 28672, 4096): (12288,),
    (8, 10240, 8192): (8192,),
    (8, 22016, 4096): (8192,),
    (8, 27648, 5120): (12288,),
    (9, 22016, 4096): (8192,),
}


# (tile order "plain" / "gate_up" / "qkv", N, K) of a matrix with a decode copy -> fewest rows
# (below 17) from which its product goes to the kernels that share X through LDS
# (csrc/gemm_rows.hip) instead of the few-rows kernels, whose waves each read X for themselves.
# Unlisted shapes: from 17 rows.
FIXED_ROWS_FROM: Dict[tuple, int] = {
    # (gate|up: measured alone the shared-X kernel wins from 1 row at these two shapes; in a
    # whole decode step at 1 and 8 rows, where its operand comes with the norm's sums of squares,
    # it does not: 318 -> 313 and 2,327 -> 2,322 tokens/s at the 8B shape)
    ("gate_up", 27648, 5120): 9,
    ("gate_up", 28672, 4096): 9,   # 12 rows: 42.3 -> 38.1 us, 16 rows: 43.7 -> 37.9
    ("qkv", 6144, 4096): 5,        # 16 rows: 18.2 -> 13.0 us
    ("qkv", 10240, 8192): 5,       # 16 rows: 45.9 -> 30.9 us
    ("qkv", 12288, 4096): 9,       # 16 rows: 25.0 -> 19.9 us
    ("qkv", 15360, 5120): 5,
}


# (tile order, N, K) -> most rows for which the product goes to csrc/gemm_rows.hip (its launch
# takes up to 128; unlisted shapes: all of them).  Measured against the vendor GEMM with the
# elementwise kernel behind it at 80 / 96 / 128 rows: q|k|v 6144 x 4096 takes 21 / 24 / 34 against
# 23 / 23 / 25 + 5 us (12288 x 4096: 26 / 27 / 36 against 30 / 33 / 34 + 5, so all rows).
FIXED_ROWS_MOST: Dict[tuple, int] = {
    ("qkv", 6144, 4096): 96,
}


class Plan:
    """The tables one engine's products are dispatched by (see the module text)."""

    def __init__(self, planes_from: Optional[dict] = None, cuts: Optional[dict] = None,
                 measure: bool = False, rows_from: Optional[dict] = None,
                 rows_most: Optional[dict] = None, rules: Optional[Rules] = None):
        self.planes_from: Dict[Tuple[int, int], int] = dict(planes_from or {})
        self.cuts: Dict[tuple, tuple] = dict(cuts or {})
        self.rows_from: Dict[tuple, int] = dict(rows_from or {})
        self.rows_most: Dict[tuple, int] = dict(rows_most or {})
        self.rules = rules or Rules()
        self.measure = bool(measure)

    @classmethod
    def fixed(cls, measure: bool = False) -> "Plan":
        return cls(FIXED_PLANES_FROM, FIXED_CUTS, measure, FIXED_ROWS_FROM, FIXED_ROWS_MOST)

    # ------------------------------------------------------------ as plain data
    def to_dict(self) -> dict:
        """JSON-able: {"planes_from": [[N, K, rows], ...], "cuts": [[key, plan], ...]}."""
        return {"planes_from": [[n, k, r] for (n, k), r in sorted(self.planes_from.items())],
                "cuts": [[list(k), list(p)] for k, p in sorted(self.cuts.items(), key=repr)],
                "rows_from": [[m, n, k, r] for (m, n, k), r in sorted(self.rows_from.items())],
                "rows_most": [[m, n, k, r] for (m, n, k), r in sorted(self.rows_most.items())],
                "rules": asdict(self.rules)}

    @classmethod
    def from_dict(cls, d: dict) -> "Plan":
        """A pinned plan: what `to_dict` gave, nothing measured."""
        return cls({(int(n), int(k)): int(r) for n, k, r in d.get("planes_from", [])},
                   {tuple(k): tuple(p) for k, p in d.get("cuts", [])}, measure=False,
                   rows_from={(str(m), int(n), int(k)): int(r) for m, n, k, r in d.get("rows_from", [])},
                   rows_most={(str(m), int(n), int(k)): int(r) for m, n, k, r in d.get("rows_most", [])},
                   rules=Rules(**{k: int(v) for k, v in d.get("rules", {}).items()}))

    def __eq__(self, other) -> bool:
        return (isinstance(other, Plan) and self.planes_from == other.planes_from
                and self.cuts == other.cuts and self.rows_from == other.rows_from
                and self.rows_most == other.rows_most and self.rules == other.rules)
