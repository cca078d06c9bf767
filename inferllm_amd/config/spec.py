"""Architecture-neutral description of a decoder: what an architecture's
configuration is translated into before anything is built.

A `ModelSpec` is plain data.  It names, layer by layer, which mixer,
feed-forward, norms and position encoding a block has (by registry name and
keyword parameters) and under which tensor names the checkpoint stores each
weight.  The order in which layers run is data too (`schedule`).  The builder in
`inferllm_amd.engine.model` turns a spec into parts; no part learns from the
spec which model it belongs to.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass
class PartSpec:
    """One part: registry name, constructor parameters, checkpoint tensor names.

    `tensors` maps the part's own parameter names (e.g. "q", "gate") to the
    tensor names of the checkpoint.
    """
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    tensors: Dict[str, str] = field(default_factory=dict)


@dataclass
class LayerSpec:
    """A block: its arrangement ("pre_norm") and the parts it is made of."""
    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    position: Optional[PartSpec] = None


@dataclass
class ScheduleEntry:
    """One run of a layer.

    `layer` indexes `ModelSpec.layers` (the weights).  `cache_line` names the
    cache storage this run uses; runs that share a number share keys and values.
    `writes_cache` False makes the run read what an earlier run of the same step
    stored on that line instead of storing its own.
    """
    layer: int
    cache_line: int
    writes_cache: bool = True


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: List[LayerSpec]
    schedule: List[ScheduleEntry]
    final_norm: PartSpec
    head: PartSpec
    bos_token_id: Optional[int] = None
    eos_token_ids: List[int] = field(default_factory=list)
    ignored_tensor_suffixes: List[str] = field(default_factory=list)

    def n_cache_lines(self) -> int:
        return 1 + max((e.cache_line for e in self.schedule), default=-1)
