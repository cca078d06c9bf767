"""RMS norm fused with the residual add that precedes it."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Norm, StepContext, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight, statistics in float32.

    src/kern/naive/naive.cpp:186-207 and src/core/op.cpp:37-47; eps is a parameter
    (the reference fixes 1e-6 / 1e-5 at src/graph/llama_like.cpp:78 and src/core/graph.h:163).
    """

    graph_safe_prompts = True

    adds_planes = True

    def __init__(self, size: int, eps: float, tensors=None):
        super().__init__(tensors)
        self.size, self.eps = int(size), float(eps)
        self.weight: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"weight": TensorWant((self.size,), init="ones_normal", keep_stored=True)}

    def load(self, tensors) -> None:
        self.weight = self._take(tensors, "weight").contiguous()

    def rms_params(self):
        return self.weight, self.eps

    def forward(self, x, delta, ctx: StepContext, row_idx=None):
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, ctx.act_dtype, row_idx)
