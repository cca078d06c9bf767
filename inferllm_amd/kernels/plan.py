"""Which of several equivalent ways a bfloat16 product takes, as data.

Some products can run in more than one way that differ in speed by shape and in rounding
only: the down projection of few rows through the residual-adding kernel or through planes
(`ops.linear_planes`), a product of many rows whole, cut along its output columns, in two
halves of its rows or filled up to 256 rows.  Which way is taken must not depend on a
stopwatch, or the same request could give other bfloat16 logits in another process.  So
the choice is a table by shape:

* `Plan.fixed()` (what an engine uses unless told otherwise): the tables below, measured once
  on an MI355X for the matrix shapes of LLaMA-2-7B, LLaMA-3-8B and LLaMA-2-70B
  (`python -m inferllm_amd.kernels.tune`), and for every other shape one rule: planes from 17
  rows on, products of many rows whole.  Nothing is ever timed.
* `Plan(measure=True)` (`Engine(tune=True)`): a shape that the tables lack is timed the first
  time it is used outside graph capture and the winner is kept; `to_dict()` gives the result,
  which `Engine(plan=...)` pins in another process.

The float32 path has one way per product and no plan.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

NEVER_BELOW = 17          # planes are not taken below 17 rows (the rule for unlisted shapes)

# (N, K) of a matrix with K >= 2 N -> fewest rows (1, 5, 9, 13 or 17) from which the planes and
# the norm that adds them take less time than the residual-adding few-rows product.
FIXED_PLANES_FROM: Dict[Tuple[int, int], int] = {
}

# (rows / 256 rounded up, N, K) -> plan of a product of at least 1024 rows and 8192 columns:
# () whole, (c,) cut of the output columns at c, ("rows", n) the rows in n equal parts.
# ("pad", rows / 32 rounded up, N, K) -> () or ("pad", 256) for products of 65 to 255 rows.
FIXED_CUTS: Dict[tuple, tuple] = {
}


class Plan:
    """The tables one engine's products are dispatched by (see the module text)."""

    def __init__(self, planes_from: Optional[dict] = None, cuts: Optional[dict] = None,
                 measure: bool = False):
        self.planes_from: Dict[Tuple[int, int], int] = dict(planes_from or {})
        self.cuts: Dict[tuple, tuple] = dict(cuts or {})
        self.measure = bool(measure)

    @classmethod
    def fixed(cls, measure: bool = False) -> "Plan":
        return cls(FIXED_PLANES_FROM, FIXED_CUTS, measure)

    # ------------------------------------------------------------ as plain data
    def to_dict(self) -> dict:
        """JSON-able: {"planes_from": [[N, K, rows], ...], "cuts": [[key, plan], ...]}."""
        return {"planes_from": [[n, k, r] for (n, k), r in sorted(self.planes_from.items())],
                "cuts": [[list(k), list(p)] for k, p in sorted(self.cuts.items(), key=repr)]}

    @classmethod
    def from_dict(cls, d: dict) -> "Plan":
        """A pinned plan: what `to_dict` gave, nothing measured."""
        return cls({(int(n), int(k)): int(r) for n, k, r in d.get("planes_from", [])},
                   {tuple(k): tuple(p) for k, p in d.get("cuts", [])}, measure=False)

    def __eq__(self, other) -> bool:
        return (isinstance(other, Plan) and self.planes_from == other.planes_from
                and self.cuts == other.cuts)
