"""A decoder built from a `ModelSpec`: embedding, blocks, the order they run in,
last norm, head.  Nothing here knows an architecture by name.

The reference's counterpart is `Graph`: a list of modules run in order
(src/core/graph.cpp:166-197) built by `construct_llm` (src/graph/llama_like.cpp:54-109).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops

from ..cache.manager import KVSpec, StateSpec
from ..config.spec import ModelSpec
from ..parts import build_part, part_class
from ..parts.base import Block, StepContext
from ..weights.loader import TensorWant


class DecoderModel:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.layers: List[Block] = []
        # position parts whose `on_embedding` hook runs on the embedded rows: one per distinct
        # position spec among the layers (layers that name the same encoding share one call)
        self.embedding_hooks: List = []
        hooked: List = []
        for ls in spec.layers:
            position = build_part("position", ls.position) if ls.position is not None else None
            if position is not None and ls.position not in hooked:
                hooked.append(ls.position)
                self.embedding_hooks.append(position)
            self.layers.append(part_class("block", ls.block)(
                mixer=build_part("mixer", ls.mixer),
                feed_forward=build_part("feed_forward", ls.feed_forward),
                mixer_norm=build_part("norm", ls.mixer_norm),
                feed_forward_norm=build_part("norm", ls.feed_forward_norm),
                position=position))
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.schedule = list(spec.schedule)
        for e in self.schedule:
            if not (0 <= e.layer < len(self.layers)):
                raise ValueError(f"schedule names layer {e.layer}; the model has {len(self.layers)}")
        writers = {}
        for e in self.schedule:
            if e.writes_cache:
                writers.setdefault(e.cache_line, e.layer)
            elif e.cache_line not in writers:
                raise ValueError(f"schedule: cache line {e.cache_line} is read before any run writes it")
        self.loaded = False
        self.graph_safe = all(getattr(p, "graph_safe", True) for p in self.every_part())
        # steps of several tokens a sequence may be replayed from graphs only if every part says so
        self.graph_safe_prompts = self.graph_safe and all(
            getattr(p, "graph_safe_prompts", False) for p in self.every_part())
        # mixers that cannot go on from their cache by more than one token a step
        self.one_token_mixers = sorted({type(l.mixer).__name__ for l in self.layers
                                        if not getattr(l.mixer, "takes_continuations", False)})

    # ------------------------------------------------------------ weights
    def wants(self) -> Dict[str, TensorWant]:
        out: Dict[str, TensorWant] = {}
        for part in [self.embedding, *self.layers, self.final_norm, self.head]:
            for name, want in part.wants().items():
                if name in out and tuple(out[name].shape) != tuple(want.shape):
                    raise ValueError(f"tensor {name!r} is wanted with two shapes: "
                                     f"{out[name].shape} and {want.shape}")
                if name in out and not out[name].optional:
                    continue
                out[name] = want
        return out

    def every_part(self) -> List:
        every = [self.embedding, self.final_norm, self.head]
        for layer in self.layers:
            every.extend([layer] + layer.parts())
        return every

    def load(self, tensors: Dict[str, torch.Tensor], decode_copies=False) -> None:
        """Hand every part its tensors.  `decode_copies`: whether the parts keep second copies of
        their matrices for the few-rows kernels (False, True or "thin")."""
        for part in self.every_part():
            part.decode_copies = decode_copies
        for part in [self.embedding, *self.layers, self.final_norm, self.head]:
            part.load(tensors)
        self.loaded = True

    # ------------------------------------------------------------ cache needs
    def kv_lines(self) -> Dict[int, KVSpec]:
        out: Dict[int, KVSpec] = {}
        for e in self.schedule:
            spec = self.layers[e.layer].mixer.kv_spec()
            if spec is None:
                continue
            if e.cache_line in out and out[e.cache_line] != spec:
                raise ValueError(f"cache line {e.cache_line} is shared by mixers with different needs")
            out[e.cache_line] = spec
        return out

    def state_lines(self) -> Dict[int, StateSpec]:
        out: Dict[int, StateSpec] = {}
        for e in self.schedule:
            spec = self.layers[e.layer].mixer.state_spec()
            if spec is not None:
                out[e.cache_line] = spec
        return out

    # ------------------------------------------------------------ compute
    def forward(self, ctx: StepContext, out_rows: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
        """Run the step's rows through every scheduled layer; logits (float32
        [len(out_rows), vocab]) for the rows asked for, or None if none is."""
        x = self.embedding.forward(ctx)
        for position in self.embedding_hooks:
            position.on_embedding(x, ctx)
        pending = None
        for i, e in enumerate(self.schedule):
            layer = self.layers[e.layer]
            if getattr(layer, "takes_next_norm", False):
                # the norm that will meet this block's output, for kernels that prepare it; none if
                # the block that follows does not say that it takes rows prepared for its norm
                # (it then finds the sum in x, or a plain tensor still to be added)
                after = self.layers[self.schedule[i + 1].layer] if i + 1 < len(self.schedule) else None
                nxt = (self.final_norm if after is None else
                       after.mixer_norm if getattr(after, "takes_prepared_rows", False) else None)
                pending = layer.forward(x, pending, ctx, e.cache_line, e.writes_cache, next_norm=nxt)
            else:
                pending = layer.forward(x, pending, ctx, e.cache_line, e.writes_cache)
        if out_rows is None or out_rows.numel() == 0:
            return None
        if isinstance(pending, ops.NormedRows):
            pending = None                       # its sum is in x already
        h = self.final_norm.forward(x, pending, ctx, row_idx=out_rows)
        return self.head.forward(h, ctx)


def expected_tensors(spec: ModelSpec) -> Dict[str, TensorWant]:
    """Checkpoint tensor name -> shape and kind, for a spec (no weights are allocated)."""
    return DecoderModel(spec).wants()
