"""The step function: one batch of sequences, either all at their first token
(whole prompts of unequal lengths) or all going on by one token; if every mixer of
the model says it can go on from what it kept by several tokens (attention does: its rows
then attend over the paged cache), also any mix of starting sequences and sequences that
go on by any number of tokens (a prompt cut into steps, a conversation's next turn).

It runs only the tokens it is given, packed as one batch, against the cache that
earlier steps left, and returns float32 logits at the places asked for.  Steps
of single tokens are replayed from a HIP graph captured per batch-size bucket;
rows that only fill a bucket up use the cache's spare slot and page and change
no result.

The reference's counterpart is `Graph::execute(tokens, logits, nr_past, prefill)`
for one sequence, with logits of the last token only and none on prefill
(src/core/graph.cpp:166-197).
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..kernels import ops
from ..parts.base import StepContext
from .model import DecoderModel


class StepError(ValueError):
    """A batch the step function does not take (mixed phases, bad token ids, ...)."""


@dataclass
class StepEntry:
    """One sequence's share of a step: its slot, its next tokens and the indices
    among these tokens whose logits are wanted."""
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)


def _bucket(n: int) -> int:
    """Rows of the graph that a decode step of n sequences is replayed from: powers of two, and
    from 16 on the sizes half way between them too (24, 48, 96, ...: the products' time grows
    with their tiles of 16 rows, so 96 rows cost less than 128)."""
    b = 1
    while b < n:
        b *= 2
    return b * 3 // 4 if b >= 32 and n <= b * 3 // 4 else b


def _length_class(n: int, limit: int) -> int:
    """The class of a decode step by its longest sequence: 1024, 2048, 4096, ... keys, at most
    the cache's limit.  How attention cuts the keys among blocks is fixed when a graph is
    captured, and what is best for 600 keys is not for 4000."""
    c = 1024
    while c < n:
        c *= 2
    return min(c, max(limit, 1))


def _ragged(lens: Sequence[int]) -> bool:
    """Whether the sequences of a decode step differ widely in length: the longest has 1,024 keys
    or more and the mean is at most 0.6 of it.  Attention then cuts the keys into more ranges, so
    that the blocks of the long sequences do not outlast everything else."""
    longest = max(lens)
    return longest >= 1024 and 10 * sum(lens) <= 6 * longest * len(lens)


class _DecodeGraph:
    """Static buffers and the captured graph for decode steps of one bucket size, one class
    of lengths and one answer to "do the lengths differ widely"."""

    def __init__(self, runner: "StepRunner", size: int, max_len: int, ragged: bool = False):
        self.size = size
        self.max_len = max_len
        self.ragged = ragged
        dev = runner.device
        self.meta = torch.zeros(4 * size, dtype=torch.int32, device=dev)   # tokens | pos | slot | len
        # host side of `meta`: pinned, so that one asynchronous copy brings a step's numbers over
        self.stage = torch.zeros(4 * size, dtype=torch.int32, pin_memory=True)
        self.stage_np = self.stage.numpy()
        self.copied = torch.cuda.Event()
        self.in_flight = False
        self.cu = torch.arange(size + 1, dtype=torch.int32, device=dev)
        self.rows = torch.arange(size, dtype=torch.int32, device=dev)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None

    def context(self, runner: "StepRunner") -> StepContext:
        n = self.size
        return StepContext(
            device=runner.device, act_dtype=runner.act_dtype, prefill=False, n_rows=n, n_seqs=n,
            tokens=self.meta[:n], row_pos=self.meta[n:2 * n], row_slot=self.meta[2 * n:3 * n],
            cu_seqlens=self.cu, seq_slot=self.meta[2 * n:3 * n], seq_len=self.meta[3 * n:],
            max_len=self.max_len, cache=runner.cache, ragged=self.ragged)


PROMPT_GRAPH_ROWS = (16, 32, 64, 96, 128, 192, 256)   # rows of the graphs that short prompt steps are replayed from
PROMPT_GRAPH_SEQS = (2, 4, 8, 16, 32)                 # and their sequences (one of them takes the padding rows)


class _PromptGraph:
    """Static buffers and the captured graph for steps of several tokens a sequence with at most
    `rows` rows in at most `seqs` - 1 sequences, of which at most 2 `seqs` rows are wanted.  Rows
    that only fill the graph up are a sequence of their own on the cache's spare slot; sequences
    that only fill it up have no rows."""

    def __init__(self, runner: "StepRunner", rows: int, seqs: int, continues: bool):
        self.rows, self.seqs, self.continues = rows, seqs, continues
        dev = runner.device
        # tokens | pos | slot (rows each) | cu (seqs + 1) | seq slot | seq len | seq start (seqs each) | wanted
        self.sizes = (rows, rows, rows, seqs + 1, seqs, seqs, seqs, 2 * seqs)
        n = sum(self.sizes)
        self.meta = torch.zeros(n, dtype=torch.int32, device=dev)
        self.stage = torch.zeros(n, dtype=torch.int32, pin_memory=True)
        self.stage_np = self.stage.numpy()
        self.copied = torch.cuda.Event()
        self.in_flight = False
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None

    def parts(self) -> List[torch.Tensor]:
        out, o = [], 0
        for n in self.sizes:
            out.append(self.meta[o:o + n])
            o += n
        return out

    def context(self, runner: "StepRunner") -> StepContext:
        p = self.parts()
        limit = runner.cache.max_seq_len
        return StepContext(
            device=runner.device, act_dtype=runner.act_dtype, prefill=True, n_rows=self.rows,
            n_seqs=self.seqs, tokens=p[0], row_pos=p[1], row_slot=p[2], cu_seqlens=p[3], seq_slot=p[4],
            seq_len=p[5], max_len=limit if self.continues else self.rows, cache=runner.cache,
            seq_start=p[6], max_rows=self.rows, continues=self.continues)

    def fill(self, runner: "StepRunner", entries: Sequence[StepEntry], starts: Sequence[int]) -> int:
        """Write the step's numbers into the pinned stage; returns the number of wanted rows."""
        spare = runner.cache.spare_slot
        wrap = max(1, min(64, runner.cache.max_seq_len))       # positions of the padding rows
        tokens: List[int] = []
        pos: List[int] = []
        slot: List[int] = []
        cu = [0]
        want: List[int] = []
        for e, start in zip(entries, starts):
            n = len(e.tokens)
            want.extend(cu[-1] + int(w) for w in e.want)
            tokens.extend(int(t) for t in e.tokens)
            pos.extend(range(start, start + n))
            slot.extend([e.slot] * n)
            cu.append(cu[-1] + n)
        pad = self.rows - len(tokens)
        idle = self.seqs - len(entries)                         # >= 1: the first takes the padding rows
        host = (tokens + [0] * pad + pos + [i % wrap for i in range(pad)] + slot + [spare] * pad
                + cu + [self.rows] * idle
                + [e.slot for e in entries] + [spare] * idle
                + [s + len(e.tokens) for e, s in zip(entries, starts)] + [max(pad, 1)] + [1] * (idle - 1)
                + [int(s) for s in starts] + [0] * idle
                + want + [0] * (2 * self.seqs - len(want)))
        self.stage_np[:] = host
        return len(want)


class StepRunner:
    """Owns the model, the cache and the step graphs; `step` is the one entry."""

    def __init__(self, model: DecoderModel, cache: CacheManager, act_dtype: torch.dtype,
                 device: torch.device, use_graphs: bool = True, plan=None):
        self.model, self.cache = model, cache
        self.plan = plan
        self.act_dtype, self.device = act_dtype, device
        self.vocab_size = model.spec.vocab_size
        self.use_graphs = (use_graphs and model.graph_safe
                           and os.environ.get("INFERLLM_NO_GRAPH", "0") != "1")
        self._graphs: Dict[tuple, _DecodeGraph] = {}
        # steps of few rows with several tokens a sequence (short prompts, a conversation's turns):
        # replayed from a graph from the second step of a shape on (the first runs eagerly: one
        # prompt does not pay for a capture), if every part of the model says it takes that
        self.use_prompt_graphs = self.use_graphs and model.graph_safe_prompts
        self._prompt_graphs: Dict[tuple, _PromptGraph] = {}
        self._prompt_uses: Dict[tuple, int] = {}

    # ------------------------------------------------------------ checks
    def _phase(self, entries: Sequence[StepEntry]) -> bool:
        """True for a step of whole prompts, False for a step of single tokens."""
        if not entries:
            raise StepError("a step needs at least one sequence")
        slots = [e.slot for e in entries]
        if len(set(slots)) != len(slots):
            raise StepError("a slot appears twice in one step")
        for e in entries:
            if len(e.tokens) == 0:
                raise StepError(f"slot {e.slot}: no tokens in this step")
            for t in e.tokens:
                if not (0 <= int(t) < self.vocab_size):
                    raise StepError(f"slot {e.slot}: token id {t} outside the vocabulary "
                                    f"of {self.vocab_size}")
            for w in e.want:
                if not (0 <= int(w) < len(e.tokens)):
                    raise StepError(f"slot {e.slot}: wanted place {w} is not among the "
                                    f"{len(e.tokens)} tokens of this step")
        starts = [self.cache.length(e.slot) == 0 for e in entries]
        if all(starts):
            return True
        if not any(starts) and all(len(e.tokens) == 1 for e in entries):
            return False
        if not self.model.one_token_mixers:
            return True            # every mixer goes on from what it kept by any number of tokens
        raise StepError("the sequences of a step must either all start at their first token "
                        "or all go on by one token: this model's "
                        f"{', '.join(self.model.one_token_mixers)} cannot go on by several")

    # ------------------------------------------------------------ the step
    @torch.no_grad()
    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None,
             borrow: bool = False) -> Optional[torch.Tensor]:
        """Run one step; float32 logits [wanted, vocab] in the order of the entries
        and of their `want`, or None when nothing is wanted.

        `device_tokens` (a step of single tokens only): int32 [len(entries)] on the device, the
        token of every entry in order, in place of the entries' own (which are placeholders
        then).  It lets a caller start the next step from tokens that were chosen on the device
        before it has read them back.

        `borrow`: the result may be a view of memory that the next step writes again (a decode
        graph's output); a caller that has used it up by then saves a copy.  Without it the
        result is the caller's to keep."""
        prefill = self._phase(entries)          # True: a step of several tokens per sequence
        if self.plan is not None:
            ops.use_plan(self.plan)
        if device_tokens is not None:
            if prefill:
                raise StepError("tokens from the device are taken by steps of single tokens only")
            if (device_tokens.dtype != torch.int32 or device_tokens.device != self.device
                    or device_tokens.shape != (len(entries),)):
                raise StepError(f"device_tokens must be int32 [{len(entries)}] on {self.device}")
        starts = [self.cache.length(e.slot) for e in entries]
        limit = self.cache.step_limit
        if (prefill and limit is not None and any(starts)
                and max(len(e.tokens) for e in entries) > limit):
            return self._in_pieces(entries, starts, limit)
        self.cache.extend_all([(e.slot, s, len(e.tokens)) for e, s in zip(entries, starts)])
        self.cache.upload(lengths=prefill)
        if prefill:
            g = self._prompt_graph_for(entries, starts)
            if g is not None:
                return self._replay_prompt(g, entries, starts, borrow)
            return self._prefill(entries, starts)
        return self._decode(entries, starts, device_tokens, borrow)

    def _prompt_graph_for(self, entries: Sequence[StepEntry], starts: Sequence[int]) -> Optional[_PromptGraph]:
        """The graph that this step of several tokens a sequence is replayed from, or None if it
        runs eagerly: more rows, sequences or wanted rows than the graphs hold, or a shape seen
        for the first time."""
        if not self.use_prompt_graphs:
            return None
        rows = sum(len(e.tokens) for e in entries)
        wanted = sum(len(e.want) for e in entries)
        if rows > PROMPT_GRAPH_ROWS[-1] or len(entries) + 1 > PROMPT_GRAPH_SEQS[-1] or wanted == 0:
            return None
        if next(b for b in PROMPT_GRAPH_ROWS if b >= rows) > self.cache.max_seq_len:
            return None         # the padding rows are a sequence too, and no sequence is that long here
        seqs = next(b for b in PROMPT_GRAPH_SEQS if b >= len(entries) + 1)
        if wanted > 2 * seqs:
            return None
        key = (next(b for b in PROMPT_GRAPH_ROWS if b >= rows), seqs, any(int(s) > 0 for s in starts))
        self._prompt_uses[key] = self._prompt_uses.get(key, 0) + 1
        g = self._prompt_graphs.get(key)
        if g is None:
            if self._prompt_uses[key] < 2:
                return None
            g = self._prompt_graphs[key] = _PromptGraph(self, *key)
        return g

    def _replay_prompt(self, g: _PromptGraph, entries: Sequence[StepEntry], starts: Sequence[int],
                       borrow: bool) -> torch.Tensor:
        if g.graph is None:
            self._capture_prompt(g)
        if g.in_flight:
            g.copied.synchronize()          # the last step's copy has left the pinned buffer
        wanted = g.fill(self, entries, starts)
        g.meta.copy_(g.stage, non_blocking=True)
        g.copied.record()
        g.in_flight = True
        g.graph.replay()
        return g.logits[:wanted] if borrow else g.logits[:wanted].clone()

    def _capture_prompt(self, g: _PromptGraph) -> None:
        """As `_capture`: one eager run of the same shapes with every row on the spare slot (one
        sequence of padding rows, the other sequences empty), then the capture."""
        g.fill(self, [], [])
        g.meta.copy_(g.stage)
        rows = g.parts()[7]
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            self.model.forward(g.context(self), rows)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            g.logits = self.model.forward(g.context(self), rows)
        g.graph = graph

    def _in_pieces(self, entries: Sequence[StepEntry], starts: Sequence[int],
                   limit: int) -> Optional[torch.Tensor]:
        """A step that reads the cache and brings some sequence more tokens than a window's ring
        of pages keeps apart, as several steps of at most `limit` tokens a sequence: a step
        stores all its keys before its rows read, and a longer one would write round the ring
        onto keys that its first rows still see.  The logits come out in the whole step's order."""
        self.cache.check_room([(e.slot, s, len(e.tokens)) for e, s in zip(entries, starts)])
        pieces, keys = [], []
        for lo in range(0, max(len(e.tokens) for e in entries), limit):
            part = []
            for i, e in enumerate(entries):
                if lo >= len(e.tokens):
                    continue
                want = [(j, int(w) - lo) for j, w in enumerate(e.want) if lo <= int(w) < lo + limit]
                part.append(StepEntry(e.slot, e.tokens[lo:lo + limit], [w for _, w in want]))
                keys.extend((i, j) for j, _ in want)
            out = self.step(part)
            if out is not None:
                pieces.append(out)
        if not pieces:
            return None
        logits = pieces[0] if len(pieces) == 1 else torch.cat(pieces, dim=0)
        order = sorted(range(len(keys)), key=keys.__getitem__)
        if order != list(range(len(keys))):
            logits = logits[torch.tensor(order, dtype=torch.long, device=self.device)]
        return logits

    def _prefill(self, entries: Sequence[StepEntry], starts: Sequence[int]) -> Optional[torch.Tensor]:
        tokens: List[int] = []
        pos: List[int] = []
        slot: List[int] = []
        cu = [0]
        want: List[int] = []
        for e, start in zip(entries, starts):
            n = len(e.tokens)
            want.extend(cu[-1] + int(w) for w in e.want)
            tokens.extend(int(t) for t in e.tokens)
            pos.extend(range(start, start + n))
            slot.extend([e.slot] * n)
            cu.append(cu[-1] + n)
        T, B = len(tokens), len(entries)
        host = torch.tensor(tokens + pos + slot + cu + [e.slot for e in entries]
                            + [s + len(e.tokens) for e, s in zip(entries, starts)]
                            + [int(s) for s in starts] + want, dtype=torch.int32)
        meta = host.to(self.device)
        o = 0
        parts = []
        for n in (T, T, T, B + 1, B, B, B, len(want)):
            parts.append(meta[o:o + n])
            o += n
        ctx = StepContext(
            device=self.device, act_dtype=self.act_dtype, prefill=True, n_rows=T, n_seqs=B,
            tokens=parts[0], row_pos=parts[1], row_slot=parts[2], cu_seqlens=parts[3],
            seq_slot=parts[4], seq_len=parts[5],
            max_len=max(s + len(e.tokens) for e, s in zip(entries, starts)),
            cache=self.cache, seq_start=parts[6], max_rows=max(len(e.tokens) for e in entries),
            continues=any(int(s) > 0 for s in starts))
        return self.model.forward(ctx, parts[7] if want else None)

    def _decode(self, entries: Sequence[StepEntry], starts: Sequence[int],
                device_tokens: Optional[torch.Tensor] = None,
                borrow: bool = False) -> Optional[torch.Tensor]:
        B = len(entries)
        size = _bucket(B) if self.use_graphs else B
        pad = size - B
        spare = self.cache.spare_slot
        host = ([int(e.tokens[0]) for e in entries] + [0] * pad
                + list(starts) + [0] * pad
                + [e.slot for e in entries] + [spare] * pad
                + [s + 1 for s in starts] + [1] * pad)          # a padding row sees one (spare) key
        wanted = [i for i, e in enumerate(entries) if len(e.want)]
        if not self.use_graphs:
            meta = torch.tensor(host, dtype=torch.int32).to(self.device)
            if device_tokens is not None:
                meta[:B].copy_(device_tokens)
            ctx = StepContext(
                device=self.device, act_dtype=self.act_dtype, prefill=False, n_rows=B, n_seqs=B,
                tokens=meta[:B], row_pos=meta[B:2 * B], row_slot=meta[2 * B:3 * B],
                cu_seqlens=torch.arange(B + 1, dtype=torch.int32, device=self.device),
                seq_slot=meta[2 * B:3 * B], seq_len=meta[3 * B:], max_len=max(starts) + 1,
                cache=self.cache, ragged=_ragged([s + 1 for s in starts]))
            rows = torch.tensor(wanted, dtype=torch.int32, device=self.device) if wanted else None
            return self.model.forward(ctx, rows)
        key = (size, _length_class(max(starts) + 1, self.cache.max_seq_len),
               _ragged([s + 1 for s in starts]))
        g = self._graphs.get(key)
        if g is None:
            g = self._graphs[key] = _DecodeGraph(self, *key)
        if g.graph is None:
            self._capture(g)
        if g.in_flight:
            g.copied.synchronize()          # the last step's copy has left the pinned buffer
        g.stage_np[:] = host
        g.meta.copy_(g.stage, non_blocking=True)
        g.copied.record()
        if device_tokens is not None:
            g.meta[:B].copy_(device_tokens)
        g.in_flight = True
        g.graph.replay()
        if not wanted:
            return None
        if wanted == list(range(B)):
            # the graph's own output, which its next replay writes again
            return g.logits[:B] if borrow else g.logits[:B].clone()
        return g.logits[torch.tensor(wanted, dtype=torch.long, device=self.device)]

    @torch.no_grad()
    def warm_up(self, batch_sizes: Sequence[int], longest: int = 1) -> int:
        """Capture the graphs that decode steps of these numbers of sequences, none longer than
        `longest` keys, would be replayed from, before the first of them comes (a capture costs
        one eager run of the step and the capture itself, tens of milliseconds).  No sequence's
        cache or state is touched.  Returns the number of graphs captured now."""
        if not self.use_graphs:
            return 0
        if self.plan is not None:
            ops.use_plan(self.plan)
        self.cache.upload(lengths=False)
        done = 0
        for n in sorted(set(int(b) for b in batch_sizes)):
            if n < 1:
                raise StepError("warm_up: batch sizes are positive")
            key = (_bucket(n), _length_class(max(int(longest), 1), self.cache.max_seq_len), False)
            g = self._graphs.get(key)
            if g is None:
                g = self._graphs[key] = _DecodeGraph(self, *key)
            if g.graph is None:
                self._capture(g)
                done += 1
        return done

    def _capture(self, g: _DecodeGraph) -> None:
        """Capture the step's graph.  Before a capture the libraries must have set themselves up,
        which takes one eager run of the same shapes: that run has every row on the cache's spare
        slot and spare page, so that no real sequence's cache or state is written twice (a part
        that updates per-sequence state is not idempotent as the store of keys is).  The capture
        itself executes nothing; the caller fills in the step's numbers and replays."""
        n = g.size
        spare = self.cache.spare_slot
        warm = torch.tensor([0] * n + [0] * n + [spare] * n + [1] * n, dtype=torch.int32)
        g.meta.copy_(warm.to(self.device))
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(side):
            self.model.forward(g.context(self), g.rows)
        torch.cuda.current_stream(self.device).wait_stream(side)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            g.logits = self.model.forward(g.context(self), g.rows)
        g.graph = graph
