"""Feed-forward parts."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorWant
from .attention import _fuse
from .base import FeedForward, StepContext, register_part


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """down( silu(h gate^T) * (h up^T) ), gate and up as one fused product.

    src/core/graph.cpp:57-79 (w1 = gate, w3 = up, w2 = down); silu(x) = x / (1 + exp(-x))
    (src/kern/naive/naive.cpp:80-89).  The reference runs silu and the multiply as two
    elementwise kernels (src/kern/gpu/kernel_gpu.cu:183-258).
    """

    graph_safe_prompts = True

    adds_residual = True
    takes_normed_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int, tensors=None):
        super().__init__(tensors)
        self.E, self.F = int(hidden_size), int(intermediate_size)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"gate": TensorWant((self.F, self.E)), "up": TensorWant((self.F, self.E)),
                "down": TensorWant((self.E, self.F))}

    def load(self, tensors) -> None:
        self.w_gate_up = ops.decode_weight(_fuse([self._take(tensors, "gate"), self._take(tensors, "up")]),
                                           "gate_up", self.decode_copies)
        self.w_down = ops.decode_weight(self._take(tensors, "down").contiguous(), "plain",
                                        self.decode_copies)

    def tunables(self):
        return (("gate_up", self.w_gate_up, {}), ("plain", self.w_down, {}))

    def forward(self, h, ctx: StepContext, residual=None, next_norm=None):
        a = ops.gate_up_silu(h, self.w_gate_up)
        if (next_norm is not None and getattr(next_norm, "adds_planes", False)
                and ops.linear_planes_fits(a, self.w_down) and ops.linear_planes_pays(a, self.w_down)):
            return ops.linear_planes(a, self.w_down)
        if residual is not None and ops.linear_add_fits(a, self.w_down, residual):
            return ops.linear_add(a, self.w_down, residual,
                                  next_norm.rms_params() if next_norm is not None else None,
                                  ctx.act_dtype)
        return ops.linear(a, self.w_down)
