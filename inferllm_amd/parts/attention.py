"""Causal self-attention with grouped kv heads over the paged cache."""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..cache.manager import KVSpec
from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Mixer, StepContext, register_part


def _fuse(ws):
    """One [sum of outs, in] matrix from several; float32 if the stored dtypes differ."""
    if len({w.dtype for w in ws}) > 1:
        ws = [w.to(torch.float32) for w in ws]
    return torch.cat(ws, dim=0).contiguous()


@register_part("mixer", "attention")
class Attention(Mixer):
    """q, k, v projections (one fused product), position encoding of q and k, the
    store of k and v, softmax(q k^T * scale + causal mask) v, output projection.

    src/core/op.cpp:412-498 with src/core/graph.h:107-111 (the `wo` product); scale
    1/sqrt(head_dim) after the dot product (op.cpp:488).  Query head h reads kv head
    h / (num_heads / num_kv_heads) (src/kern/naive/naive.cpp:576-604).  `window`
    keeps only the last `window` keys visible; `softmax_scale` replaces the default.
    Whole prompts attend over the step's own rows; single tokens, and rows that go on from
    tokens of earlier steps, over the cache.
    """

    graph_safe_prompts = True

    adds_residual = True
    takes_normed_rows = True

    # A step of several tokens may go on from keys the cache holds (a prompt cut into steps, a
    # conversation's next turn): its rows then attend over the paged cache.  With a window the
    # cache keeps a ring of pages; the step function cuts a step that would write round the ring
    # into what its own first rows still read (`CacheManager.step_limit`).
    takes_continuations = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 window: Optional[int] = None, softmax_scale: Optional[float] = None, tensors=None):
        super().__init__(tensors)
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if head_dim > 256:
            raise ValueError(f"head_dim {head_dim} is beyond the attention kernels' limit of 256")
        self.E, self.nh, self.nkv, self.hd = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.window = int(window) if window else None
        self.scale = float(softmax_scale) if softmax_scale else 1.0 / math.sqrt(self.hd)
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"q": TensorWant((self.nh * self.hd, self.E)),
                "k": TensorWant((self.nkv * self.hd, self.E)),
                "v": TensorWant((self.nkv * self.hd, self.E)),
                "o": TensorWant((self.E, self.nh * self.hd))}

    def kv_spec(self) -> KVSpec:
        return KVSpec.keys_values(self.nkv, self.hd, self.window)

    def load(self, tensors) -> None:
        # the decode copy of q|k|v follows the tiles of the position encoding's fused kernel, if it
        # has one; else plain tiles, which the few-rows product reads
        mode = self.position.qkv_tile_mode(self.hd) if self.position is not None else "plain"
        geometry = dict(nh=self.nh, nkv=self.nkv, hd=self.hd) if mode == "qkv" else {}
        self.w_qkv = ops.decode_weight(_fuse([self._take(tensors, n) for n in ("q", "k", "v")]),
                                       mode, self.decode_copies, **geometry)
        self.w_o = ops.decode_weight(self._take(tensors, "o").contiguous(), "plain",
                                     self.decode_copies)

    def tunables(self):
        return (("qkv", self.w_qkv, dict(nh=self.nh, nkv=self.nkv, hd=self.hd)),
                ("plain", self.w_o, {}))

    def forward(self, h, ctx: StepContext, line, writes_cache, position, residual=None,
                next_norm=None):
        nh, nkv, hd = self.nh, self.nkv, self.hd
        kc, vc, group = ctx.cache.kv_line(line)
        window = self.window or 0
        if writes_cache:
            if position is not None:
                qkv = position.project_qkv(h, self.w_qkv, ctx, nh, nkv, hd, kc, vc, group)
            else:
                qkv = ops.linear(h, self.w_qkv)
                ops.rope_store(qkv, None, 0, 0, ctx.row_pos, ctx.row_slot,
                               ctx.cache.slot_len if ctx.prefill else None, kc, vc, group.table,
                               group.page_size, group.ring, nh, nkv, hd)
            if ctx.prefill:
                ctx.exchange[("kv_rows", line)] = qkv      # for runs that read this cache line
        else:
            # keys and values are those an earlier run of this step stored on the line: only q
            # is projected and encoded (as packed rows with no kv heads)
            q = ops.linear(h, ops.plain_weight(self.w_qkv)[: nh * hd])
            if position is not None:
                position.on_qkv(q, ctx, nh, 0, hd, None, None, None)
            if ctx.prefill and not ctx.continues:
                kv = ctx.exchange[("kv_rows", line)][:, nh * hd:]
            else:
                kv = q.new_zeros((q.shape[0], 2 * nkv * hd))   # read from the cache
            qkv = torch.cat([q, kv], dim=1)
        if ctx.prefill and ctx.continues:
            # some sequence goes on from tokens of earlier steps: over the cache, which holds
            # this step's keys and values too by now
            o = ops.attn_prefill_paged(qkv, ctx.cu_seqlens, ctx.seq_slot, ctx.seq_start, kc, vc,
                                       group.table, group.page_size, group.ring, ctx.n_seqs,
                                       ctx.max_rows, nh, nkv, hd, self.scale, window)
        elif ctx.prefill:
            o = ops.attn_prefill(qkv, ctx.cu_seqlens, ctx.n_seqs, ctx.max_len, nh, nkv, hd,
                                 self.scale, window)
        else:
            longest = min(ctx.max_len, window) if window else ctx.max_len
            nsplit, waves = ops.decode_splits(ctx.n_seqs, nkv, longest, nh, hd,
                                              ragged=ctx.ragged and not window)
            o = ops.attn_decode(qkv, kc, vc, group.table, group.page_size, group.ring,
                                ctx.seq_slot, ctx.seq_len, nh, nkv, hd, self.scale, window,
                                nsplit, waves)
        if (next_norm is not None and getattr(next_norm, "adds_planes", False)
                and ops.linear_planes_fits(o, self.w_o) and ops.linear_planes_pays(o, self.w_o)):
            return ops.linear_planes(o, self.w_o)
        if residual is not None and ops.linear_add_fits(o, self.w_o, residual):
            return ops.linear_add(o, self.w_o, residual,
                                  next_norm.rms_params() if next_norm is not None else None,
                                  ctx.act_dtype)
        return ops.linear(o, self.w_o)
