"""The two ends of a decoder: token embedding and the head that gives logits."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..kernels import ops
from ..weights.loader import TensorWant
from .base import Embedding, Head, StepContext, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Embedding):
    """Row copy, no scaling (src/kern/naive/naive.cpp:43-54); rows become float32."""

    graph_safe_prompts = True

    def __init__(self, vocab_size: int, hidden_size: int, tensors=None):
        super().__init__(tensors)
        self.V, self.E = int(vocab_size), int(hidden_size)
        self.weight: Optional[torch.Tensor] = None

    def shapes(self) -> Dict[str, TensorWant]:
        return {"weight": TensorWant((self.V, self.E))}

    def load(self, tensors) -> None:
        self.weight = self._take(tensors, "weight").contiguous()

    def forward(self, ctx: StepContext):
        return ops.embed(ctx.tokens, self.weight)


@register_part("head", "lm_head")
class LMHead(Head):
    """logits = h . W^T in float32, for the rows asked for only.

    src/core/graph.cpp:117-141 and src/core/op.cpp:230-274 (the reference takes the
    last row only).  `tied_fallback` names the tensor used when the head's own is
    absent from the checkpoint (tied embeddings).
    """

    graph_safe_prompts = True

    def __init__(self, hidden_size: int, vocab_size: int, tied_fallback: Optional[str] = None,
                 tensors=None):
        super().__init__(tensors)
        self.E, self.V = int(hidden_size), int(vocab_size)
        self.tied_fallback = tied_fallback
        self.weight: Optional[torch.Tensor] = None

    def wants(self) -> Dict[str, TensorWant]:
        out = {self.tensors["weight"]: TensorWant((self.V, self.E),
                                                  optional=self.tied_fallback is not None)}
        if self.tied_fallback is not None:
            out[self.tied_fallback] = TensorWant((self.V, self.E))
        return out

    def load(self, tensors) -> None:
        own = self.tensors["weight"]
        self.weight = ops.decode_weight(
            (tensors[own] if own in tensors else tensors[self.tied_fallback]).contiguous(),
            "plain", self.decode_copies)

    def forward(self, h, ctx: StepContext):
        return ops.linear(h, self.weight, out_dtype=torch.float32)
