"""Position encodings.  Every packed row carries its absolute position; an
encoding turns it into a change of q and k (rotary) or does nothing."""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from ..kernels import ops
from .base import PositionEncoding, StepContext, register_part

_TABLES: Dict[Tuple, torch.Tensor] = {}


def rotary_table(theta: float, rotary_dim: int, max_positions: int, device) -> torch.Tensor:
    """cos and sin of p * theta^(-2i/rotary_dim), float32 [max_positions, rotary_dim/2, 2].

    Angles are formed in double precision, as the reference's plain kernel does
    (src/kern/naive/naive.cpp:396-399), and rounded once.  Tables are shared by all
    layers with the same constants.
    """
    key = (float(theta), int(rotary_dim), int(max_positions), str(device))
    t = _TABLES.get(key)
    if t is None:
        i = torch.arange(rotary_dim // 2, dtype=torch.float64)
        inv = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * i / rotary_dim)
        ang = torch.arange(max_positions, dtype=torch.float64)[:, None] * inv[None, :]
        t = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).to(torch.float32).to(device)
        _TABLES[key] = t.contiguous()
        t = _TABLES[key]
    return t


@register_part("position", "rotary")
class Rotary(PositionEncoding):
    """Rotation of pairs of q and k by position-dependent angles.

    pairing "half": pairs (i, i + head_dim/2) (src/kern/naive/naive.cpp:389-414, the
    LLaMA-2 graph's RotMode::ModelRotHalf); "interleaved": pairs (2i, 2i+1)
    (naive.cpp:415-440).  theta, rotary_dim and max_positions are parameters.
    """

    graph_safe_prompts = True

    def __init__(self, head_dim: int, rotary_dim: int, theta: float, pairing: str,
                 max_positions: int, tensors=None):
        super().__init__(tensors)
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"unknown rotary pairing {pairing!r}")
        if rotary_dim % 2 or rotary_dim > head_dim or rotary_dim <= 0:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and within head_dim {head_dim}")
        self.head_dim, self.rotary_dim = int(head_dim), int(rotary_dim)
        self.theta, self.pairing, self.max_positions = float(theta), pairing, int(max_positions)

    def table(self, device) -> torch.Tensor:
        return rotary_table(self.theta, self.rotary_dim, self.max_positions, device)

    def on_qkv(self, qkv, ctx: StepContext, nh, nkv, hd, kcache, vcache, group) -> None:
        ops.rope_store(qkv, self.table(ctx.device), self.rotary_dim,
                       0 if self.pairing == "half" else 1, ctx.row_pos, ctx.row_slot,
                       ctx.cache.slot_len if ctx.prefill else None, kcache, vcache,
                       group.table if group is not None else None,
                       group.page_size if group is not None else 1,
                       group.ring if group is not None else 0, nh, nkv, hd)


    def qkv_tile_mode(self, head_dim: int) -> str:
        # the fused product + rotation + store kernels pair a row with its partner head_dim / 2 on
        fused = self.pairing == "half" and self.rotary_dim == head_dim and head_dim % 16 == 0
        return "qkv" if fused else "plain"

    def project_qkv(self, h, w_qkv, ctx: StepContext, nh, nkv, hd, kcache, vcache, group):
        if (not ctx.prefill and kcache is not None and self.pairing == "half"
                and self.rotary_dim == hd and ops.qkv_rope_store_fits(h, w_qkv, hd)
                and kcache.dtype == torch.bfloat16):
            return ops.qkv_rope_store(h, w_qkv, self.table(ctx.device), ctx.row_pos, ctx.row_slot,
                                      kcache, vcache, group.table, group.page_size, group.ring,
                                      nh, nkv, hd)
        return super().project_qkv(h, w_qkv, ctx, nh, nkv, hd, kcache, vcache, group)


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No encoding: q and k stay as they are; k and v are still stored."""

    graph_safe_prompts = True

    def on_qkv(self, qkv, ctx: StepContext, nh, nkv, hd, kcache, vcache, group) -> None:
        ops.rope_store(qkv, None, 0, 0, ctx.row_pos, ctx.row_slot,
                       ctx.cache.slot_len if ctx.prefill else None, kcache,
                       vcache, group.table if group is not None else None,
                       group.page_size if group is not None else 1,
                       group.ring if group is not None else 0, nh, nkv, hd)
