"""Interfaces of the parts a decoder is put together from, and their registries.

A part is built from keyword parameters (its sizes and constants) and a map from
its own parameter names to checkpoint tensor names.  It says which tensors it
wants (`wants`), takes them (`load`) and computes (`forward`).  No part knows
which model it is in: everything it needs comes through its constructor and the
`StepContext` of the step.

Five kinds: mixer (attention and whatever else mixes tokens), feed-forward, norm,
position encoding, block (the arrangement of the other four around the residual
stream); plus the embedding and the head at the model's ends.  Each kind has a
registry from a name to a class, so another part is added by registering a class,
without touching the files here.  The reference assembles its graph the same way
from ops with constants as constructor arguments (src/graph/llama_like.cpp:54-109).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional

import torch

from ..cache.manager import CacheManager, KVSpec, StateSpec
from ..weights.loader import TensorWant


@dataclass
class StepContext:
    """What a step hands to every part.

    Rows are the step's tokens, packed sequence after sequence.  All index tensors
    are int32 on the device.  `prefill` steps carry whole prompts that start at
    position 0; other steps carry one token per sequence.
    """
    device: torch.device
    act_dtype: torch.dtype            # dtype of activations between kernels (residual is float32)
    prefill: bool
    n_rows: int
    n_seqs: int
    tokens: torch.Tensor              # [rows]
    row_pos: torch.Tensor             # [rows] absolute position of each row
    row_slot: torch.Tensor            # [rows] cache slot of each row
    cu_seqlens: torch.Tensor          # [seqs + 1] row offsets of the sequences
    seq_slot: torch.Tensor            # [seqs]
    seq_len: torch.Tensor             # [seqs] length of each sequence after this step
    max_len: int                      # longest sequence after this step (host number)
    cache: CacheManager
    # steps of several tokens a sequence (`prefill`): where each sequence's rows begin, and whether
    # any begins beyond position 0 (the step goes on from what the cache and the states hold)
    seq_start: Optional[torch.Tensor] = None     # [seqs] position of the sequence's first row
    max_rows: int = 0                 # most rows a sequence brings (host number)
    continues: bool = False
    # a step of single tokens whose sequences differ widely in length (their mean is at most 0.6
    # of the longest): work that is cut evenly by sequence is then uneven by block
    ragged: bool = False
    exchange: Dict[Any, Any] = field(default_factory=dict)   # between runs of layers in one step


class Part:
    """Base of all parts: parameter names -> checkpoint names in `self.tensors`.

    `graph_safe`: the part's forward only launches work on the current stream (no host
    synchronisation, no host reads of device data), so decode steps that contain it may
    be captured into a HIP graph.  A part that reads device data on the host sets it False.

    `graph_safe_prompts`: the same holds for steps of several tokens a sequence, which are then
    replayed from graphs too when they have few rows.  Such a step has the graph's shapes, not its
    own: `ctx.n_rows`, `ctx.n_seqs`, `ctx.max_len` and `ctx.max_rows` are upper bounds, the rows
    that fill the graph up are a sequence of their own on the cache's spare slot, and sequences
    that fill it up have no rows.  A part has to say that it takes this; the library's own do.
    """
    graph_safe = True
    graph_safe_prompts = False
    # A short cut between a block's parts for steps of few rows (False: the plain protocol, which
    # every part supports).  A mixer or feed-forward with `adds_residual` takes
    # `forward(..., residual=x, next_norm=norm)` and may add its result to the float32 residual
    # rows `x` in its last kernel; it then returns None, or, if that kernel could also prepare
    # the norm that follows (`next_norm.rms_params()`), `ops.NormedRows` for the next part.
    # A part with `takes_normed_rows` accepts `ops.NormedRows` as its `h`.
    adds_residual = False
    takes_normed_rows = False
    # Set by the model before `load`: whether the engine wants second copies of the matrices in
    # the few-rows kernels' tile order (False, True or "thin"; see `ops.decode_weight`).
    decode_copies = False

    def __init__(self, tensors: Optional[Dict[str, str]] = None):
        self.tensors: Dict[str, str] = dict(tensors or {})

    def shapes(self) -> Dict[str, TensorWant]:
        """Own parameter name -> what is wanted of it."""
        return {}

    def wants(self) -> Dict[str, TensorWant]:
        """Checkpoint tensor name -> what is wanted of it."""
        return {self.tensors[p]: w for p, w in self.shapes().items()}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Take the wanted tensors out of `tensors` (checkpoint name -> tensor on the device)."""

    def _take(self, tensors: Dict[str, torch.Tensor], param: str) -> torch.Tensor:
        return tensors[self.tensors[param]]

    def tunables(self):
        """The part's products that have several equivalent ways, for whoever times them (an
        engine built with `tune=True`, `kernels.tune`): tuples (kind, weight, geometry), kind
        "plain" (a matrix of ordinary products), "gate_up" (a fused gate|up matrix in its fused
        kernel's tile order) or "qkv" (a fused q|k|v matrix likewise; geometry `nh`, `nkv`, `hd`).
        A part that lists nothing is never timed and takes the rule for unlisted shapes."""
        return ()


class Mixer(Part):
    # The position encoding of the mixer's block, set by the block before `load` (None: none).
    position = None
    # True: in a step of several tokens per sequence (`ctx.prefill`) the mixer also serves
    # sequences that already hold tokens, reading what it kept of them (rows then start at
    # `ctx.row_pos`, not at 0).  False: such a step must start every sequence at its first
    # token; the step function refuses anything else and names the mixer.
    takes_continuations = False

    def kv_spec(self) -> Optional[KVSpec]:
        """Keys/values the mixer keeps per token, or None."""
        return None

    def state_spec(self) -> Optional[StateSpec]:
        """Fixed-size state the mixer keeps per sequence, or None."""
        return None

    def forward(self, h: torch.Tensor, ctx: StepContext, line: int, writes_cache: bool,
                position: Optional["PositionEncoding"]) -> torch.Tensor:
        """h [rows, hidden] (activation dtype) -> what is added to the residual stream."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError


class Norm(Part):
    # True: `forward` also takes `delta` as float32 planes [S, rows, width] that it adds in order
    # (a product whose K was split, `ops.linear_planes`).  Parts hand planes only to a norm that
    # says so.
    adds_planes = False

    def rms_params(self):
        """(weight, eps) if the norm is a plain RMS norm that a product's kernel may take over
        (see `Part.adds_residual`), else None."""
        return None

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], ctx: StepContext,
                row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Add `delta` to the float32 residual rows `x` (in place unless `row_idx`
        picks rows) and return the normed rows in the activation dtype."""
        raise NotImplementedError


class PositionEncoding(Part):
    def on_embedding(self, x: torch.Tensor, ctx: StepContext) -> None:
        """Hook for encodings that act on the embedded rows (in place)."""

    def on_qkv(self, qkv: torch.Tensor, ctx: StepContext, nh: int, nkv: int, hd: int,
               kcache, vcache, group) -> None:
        """Encode q and k of packed rows in place and store k, v in the cache (if given)."""
        raise NotImplementedError

    def qkv_tile_mode(self, head_dim: int) -> str:
        """The tile order in which `project_qkv` wants the decode copy of the fused q|k|v matrix
        (`ops.tile_rows`): "plain" unless the encoding has a fused kernel with tiles of its own."""
        return "plain"

    def project_qkv(self, h: torch.Tensor, w_qkv: torch.Tensor, ctx: StepContext, nh: int,
                    nkv: int, hd: int, kcache, vcache, group) -> torch.Tensor:
        """Packed rows [q | k | v] = h . w_qkv^T, encoded, k and v stored.  An encoding may
        override this with a fused kernel; in a step of single tokens the k and v parts of the
        returned rows need not be filled (they are read from the cache)."""
        from ..kernels import ops
        qkv = ops.linear(h, w_qkv)
        self.on_qkv(qkv, ctx, nh, nkv, hd, kcache, vcache, group)
        return qkv


class Block(Part):
    # `takes_next_norm`: `forward` also takes `next_norm=`, the norm that will meet what the block
    # hands on, and may hand on None (the sum is in x already) or `ops.NormedRows` prepared for it.
    # `takes_prepared_rows`: the block accepts `ops.NormedRows` as `pending`.  Both False: the
    # plain protocol, `pending` is None or a tensor (or planes, if its first norm adds planes).
    takes_next_norm = False
    takes_prepared_rows = False

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm,
                 feed_forward_norm: Norm, position: Optional[PositionEncoding]):
        super().__init__()
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm
        self.position = position

    def parts(self) -> List[Part]:
        ps = [self.mixer, self.feed_forward, self.mixer_norm, self.feed_forward_norm]
        return ps + ([self.position] if self.position is not None else [])

    def wants(self) -> Dict[str, TensorWant]:
        out: Dict[str, TensorWant] = {}
        for p in self.parts():
            out.update(p.wants())
        return out

    def load(self, tensors) -> None:
        self.mixer.position = self.position      # a mixer may lay its matrices out for the encoding
        for p in self.parts():
            p.load(tensors)

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext,
                line: int, writes_cache: bool) -> Optional[torch.Tensor]:
        """x: float32 residual rows, updated in place; `pending` is what the previous
        block still has to add.  Returns what this block leaves to be added."""
        raise NotImplementedError


class Embedding(Part):
    def forward(self, ctx: StepContext) -> torch.Tensor:
        """float32 residual rows [rows, hidden] for ctx.tokens."""
        raise NotImplementedError


class Head(Part):
    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        """Normed rows -> float32 logits [rows, vocab]."""
        raise NotImplementedError


# ---------------------------------------------------------------- registries
_KINDS = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
_REGISTRY: Dict[str, Dict[str, type]] = {k: {} for k in _KINDS}


def register_part(kind: str, name: str) -> Callable[[type], type]:
    """Class decorator: `@register_part("mixer", "attention")`."""
    if kind not in _REGISTRY:
        raise KeyError(f"unknown kind of part {kind!r}; kinds: {_KINDS}")

    def deco(cls: type) -> type:
        _REGISTRY[kind][name] = cls
        return cls
    return deco


def part_class(kind: str, name: str) -> type:
    try:
        return _REGISTRY[kind][name]
    except KeyError:
        raise KeyError(f"no {kind} named {name!r}; registered: {sorted(_REGISTRY[kind])}") from None


def build_part(kind: str, spec) -> Part:
    """A part from a `PartSpec` (registry name, parameters, tensor names)."""
    return part_class(kind, spec.kind)(tensors=spec.tensors, **spec.params)
