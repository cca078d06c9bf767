"""The generation loop above the step function.

Requests are served in batches, one after another: a batch takes as many of the
waiting prompts (in order) as slots and cache room allow, runs all its prompts
(unequal lengths) in one step, then one token per live sequence per step.  A
sequence ends at a stop token, at its `max_new_tokens`, or when it reaches the
longest length the cache allows; it then leaves the batch (its slot is given
back) while the others go on.  No request joins a batch that has started.

When the sampler can hand its tokens on the device (`draw`), the loop runs one step ahead:
the next step starts from the tokens on the device while the host still waits for their copy,
so the GPU does not idle while the host decides.  Ends by count (`max_new_tokens`, the context
limit) are known beforehand; a sequence that drew a stop token has one more step on its way,
whose result is dropped.  A draw that looks at the tokens before it (the repeat penalty) gets
the newest one, which the host has not read yet, from the device as well (`latest`).

With `max_step_tokens` the prompts of a batch are fed in several steps of at most that many
tokens (`plan_prefill`): a long prompt, or many prompts, need not fit one step's activations.
A step then holds sequences that go on beside sequences that start, which the step function
takes from models whose mixers can go on by several tokens.

A conversation (`engine/session.py`) is a batch of one whose slot the caller owns: `run_turn`
feeds a turn's tokens after what the slot already holds and decodes the answer through the same
loop, so it runs ahead too.  A stop token then has its void step behind it, which fed the token
into the cache: the slot is taken back by that one token (`rewind_slot`), because the token that
ends a turn is never run (application/chat.cpp:264-268).

The loop only decides; computing is behind a few callables, so its decisions can
be tested without a GPU.  The reference's loop is `application/chat.cpp:221-275`
over `ModelImp::decode_iter` (src/core/model_imp.cpp:55-79): one sequence, ended by
token 2 or a full context, `n_predict` declared but unused (chat.cpp:23).
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..cache.manager import round_up
from ..sampling.params import SamplingParams, request_seed
from .step import StepEntry


@dataclass
class GenerationStats:
    prompt_tokens: int = 0
    generated_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    decode_steps: int = 0
    batches: int = 0
    # a stopwatch over the last decode steps of a run, for measurements (`GenerationLoop.time_after`)
    timed_seconds: float = 0.0
    timed_steps: int = 0

    def summary(self) -> str:
        """Like the reference's decode_summary (src/core/model_imp.cpp:133-141), but the
        decode rate counts generated tokens only."""
        pf = self.prompt_tokens / self.prefill_seconds if self.prefill_seconds > 0 else 0.0
        decoded = max(0, self.generated_tokens - self.batches)   # first tokens come from prefill
        dc = decoded / self.decode_seconds if self.decode_seconds > 0 else 0.0
        return (f"prefill: {self.prompt_tokens} tokens, {self.prefill_seconds * 1e3:.1f} ms, "
                f"{pf:.1f} token/s\n"
                f"decode:  {self.generated_tokens} tokens in {self.decode_steps} steps, "
                f"{self.decode_seconds * 1e3:.1f} ms, {dc:.1f} token/s")


def plan_prefill(prompt_lens: Sequence[int], limit: int) -> List[List[tuple]]:
    """The steps that feed prompts of these lengths with at most `limit` tokens a step: lists of
    (place in the batch, first token, number of tokens).  Prompts are fed in order; a step takes
    the rest of the prompt that is under way, then goes on with the next ones while it has
    room."""
    if limit < 1:
        raise ValueError(f"max_step_tokens must be at least 1, got {limit}")
    done = [0] * len(prompt_lens)
    steps: List[List[tuple]] = []
    while any(d < n for d, n in zip(done, prompt_lens)):
        room, step = limit, []
        for i, n in enumerate(prompt_lens):
            if done[i] < n and room > 0:
                take = min(n - done[i], room)
                step.append((i, done[i], take))
                done[i] += take
                room -= take
        steps.append(step)
    return steps


@dataclass
class _Live:
    index: int                 # request index in the call
    slot: int
    feed: Sequence[int]        # the tokens to run before the first draw (the prompt, or a turn)
    seed: int
    base: int = 0              # tokens the slot held before `feed`
    out: List[int] = field(default_factory=list)
    history: List[int] = field(default_factory=list)
    drawn: int = 0             # tokens drawn and read in this call (the pipelined loop counts with it)
    dead: bool = False
    counter0: int = 0          # draws the sequence had behind it before this call
    owned: bool = True         # the loop took the slot and gives it back
    why: Optional[str] = None  # why it ended
    void_fed: bool = False     # a void step ran the token that ended it

    @property
    def prompt_len(self) -> int:
        """Tokens of the sequence when its first token is drawn."""
        return self.base + len(self.feed)


class GenerationLoop:
    """`step(entries) -> logits`, `sample(logits, seeds, counters, histories) -> ids`,
    `alloc_slot() -> slot`, `free_slot(slot)`; limits of the cache as numbers.

    `draw(logits, seeds, counters, histories, latest)` (optional): like `sample`, but returns an
    object with `.device` (the tokens where the step function can take them from: `step(entries,
    device_tokens=...)`), `.pick(rows)` (those of some rows) and `.tokens()` (the host list,
    waiting if need be); `latest` are the newest tokens, still unread, in the same form, and
    `histories` the ones before them.  With it the loop runs one step ahead.

    What `step` returns need only last until the next step: a row that is wanted longer (the
    last-token logits of a prompt fed in several steps) is taken out with `keep` at once."""

    def __init__(self, step: Callable, sample: Callable, alloc_slot: Callable[[], int],
                 free_slot: Callable[[int], None], max_batch: int, max_tokens: int,
                 max_seq_len: int, page_size: int = 64, sync: Optional[Callable[[], None]] = None,
                 on_token: Optional[Callable[[int, int], None]] = None,
                 draw: Optional[Callable] = None, max_step_tokens: Optional[int] = None,
                 keep: Optional[Callable] = None, join: Optional[Callable] = None,
                 rewind_slot: Optional[Callable[[int, int], None]] = None):
        """`max_step_tokens`: most tokens the prompts' steps may hold (None: a batch's prompts in
        one step).  `keep(logits, row)` then takes one row out of a step's logits as something
        that outlives the step (default: `logits[row]`, for logits that are lists), and
        `join(rows)` puts the sequences' rows, in batch order, together in the step function's
        form (default: a list).  `rewind_slot(slot, n)`: take the last n tokens of a slot back
        (for `run_turn` with `draw`)."""
        self.step, self.sample = step, sample
        self.draw = draw
        self.max_step_tokens = max_step_tokens
        self.keep = keep or (lambda logits, row: logits[row])
        self.join = join or list
        self.alloc_slot, self.free_slot = alloc_slot, free_slot
        self.rewind_slot = rewind_slot
        self.max_batch, self.max_tokens, self.max_seq_len = max_batch, max_tokens, max_seq_len
        self.page_size = page_size
        self.sync = sync or (lambda: None)
        self.on_token = on_token            # called with (request index, token) as tokens are kept
        self.stats = GenerationStats()
        # measurements: after this many decode steps of a batch the loop waits for the device once
        # and `stats.timed_seconds` / `timed_steps` count from there to the batch's end (None: off)
        self.time_after: Optional[int] = None
        self._mark: Optional[tuple] = None

    # ------------------------------------------------------------ decisions
    def room_needed(self, prompt_len: int, max_new_tokens: int) -> int:
        """Cache room to set aside for a request: the tokens it can come to hold, in whole pages.
        The last generated token is never fed back, so it needs no room."""
        most = min(self.max_seq_len, prompt_len + max(0, max_new_tokens - 1))
        return round_up(max(most, 1), self.page_size)

    def next_batch(self, waiting: Sequence[int], prompt_lens: Sequence[int],
                   max_new_tokens: int) -> List[int]:
        """The prefix of `waiting` (request indices) that fits slots and cache room."""
        batch: List[int] = []
        room = 0
        for i in waiting:
            need = self.room_needed(prompt_lens[i], max_new_tokens)
            if len(batch) >= self.max_batch or room + need > self.max_tokens:
                break
            batch.append(i)
            room += need
        if not batch:
            i = waiting[0]
            raise ValueError(f"request {i} ({prompt_lens[i]} prompt tokens, {max_new_tokens} new) "
                             f"needs more cache room than there is ({self.max_tokens} tokens)")
        return batch

    @staticmethod
    def ended(token: int, n_generated: int, total_len: int, stop_ids, max_new_tokens: int,
              max_seq_len: int) -> Optional[str]:
        """Why a sequence ends after drawing `token`, or None if it goes on.
        total_len: tokens of the sequence, the drawn one included."""
        if token in stop_ids:
            return "stop"
        if n_generated >= max_new_tokens:
            return "length"
        if total_len > max_seq_len:
            return "context"        # the drawn token could not be fed back
        return None

    def _prefill(self, live: Sequence[_Live]):
        """The batch's prompts through the step function; the logits at every prompt's last
        token, in batch order."""
        lens = [len(s.feed) for s in live]
        if self.max_step_tokens is None or sum(lens) <= self.max_step_tokens:
            return self.step([StepEntry(s.slot, s.feed, [len(s.feed) - 1]) for s in live])
        rows: List = [None] * len(live)
        for step in plan_prefill(lens, self.max_step_tokens):
            entries, owners = [], []
            for i, start, n in step:
                s = live[i]
                ends = start + n == len(s.feed)
                entries.append(StepEntry(s.slot, s.feed[start:start + n], [n - 1] if ends else []))
                if ends:
                    owners.append(i)
            logits = self.step(entries)
            for row, i in enumerate(owners):
                rows[i] = self.keep(logits, row)    # now: the next step may write where they lie
        return self.join(rows)

    def _release(self, s: _Live) -> None:
        """A sequence leaves the batch: its slot goes back, or, if the caller owns it, the void
        step's token is taken out of it."""
        if s.slot < 0:
            return
        if s.owned:
            self.free_slot(s.slot)
        elif s.void_fed:
            self.rewind_slot(s.slot, 1)
            s.void_fed = False
        s.slot = -1

    # ------------------------------------------------------------ the loop
    def run(self, prompts: Sequence[Sequence[int]], params: SamplingParams, max_new_tokens: int,
            stop_token_ids: Sequence[int] = (), include_stop: bool = False) -> List[List[int]]:
        for i, p in enumerate(prompts):
            if len(p) == 0:
                raise ValueError(f"request {i}: empty prompt")
            if len(p) > self.max_seq_len:
                raise ValueError(f"request {i}: prompt of {len(p)} tokens is longer than the "
                                 f"cache allows ({self.max_seq_len})")
        stop_ids = set(int(t) for t in stop_token_ids)
        results: List[List[int]] = [[] for _ in prompts]
        if max_new_tokens <= 0:
            return results
        waiting = list(range(len(prompts)))
        lens = [len(p) for p in prompts]
        while waiting:
            batch = self.next_batch(waiting, lens, max_new_tokens)
            waiting = waiting[len(batch):]
            live: List[_Live] = []
            try:
                for i in batch:
                    live.append(_Live(index=i, slot=self.alloc_slot(), feed=prompts[i],
                                      seed=request_seed(params.seed, i),
                                      history=[int(t) for t in prompts[i]]))
                self._serve(live, max_new_tokens, stop_ids, include_stop)
            finally:
                for s in live:
                    self._release(s)
            for s in live:
                results[s.index] = s.out
        return results

    def run_turn(self, slot: int, held: int, tokens: Sequence[int], history: List[int], seed: int,
                 draws_before: int, max_new_tokens: int, stop_token_ids: Sequence[int] = (),
                 include_stop: bool = False) -> _Live:
        """One sequence in a slot that the caller owns and that holds `held` tokens: run `tokens`
        after them and generate.  `history` (every token of the sequence so far, `tokens`
        included) is appended to as tokens are read; `draws_before` continues the sampler's
        counter.  The slot is left holding everything that was run: all of the answer but its
        last token (`why` "length" or "context": that one is still to be run) or but the stop
        token (`why` "stop").  Returns the sequence's record (`out`, `why`, `drawn`)."""
        if len(tokens) == 0:
            raise ValueError("a turn needs at least one token")
        if self.draw is not None and self.rewind_slot is None:
            raise ValueError("run_turn with `draw` needs `rewind_slot`")
        s = _Live(index=0, slot=slot, feed=tokens, seed=seed, base=held, history=history,
                  counter0=draws_before, owned=False)
        try:
            if max_new_tokens > 0:
                self._serve([s], max_new_tokens, set(int(t) for t in stop_token_ids), include_stop)
        finally:
            self._release(s)
        return s

    def _serve(self, live: List[_Live], max_new_tokens: int, stop_ids, include_stop: bool) -> None:
        self.stats.batches += 1
        self.sync()
        t0 = time.perf_counter()
        logits = self._prefill(live)
        first = (self.draw(logits, [s.seed for s in live], [s.counter0 for s in live],
                           [s.history for s in live], None) if self.draw is not None else
                 self.sample(logits, [s.seed for s in live], [s.counter0 for s in live],
                             [s.history for s in live]))
        self.sync()
        self.stats.prefill_seconds += time.perf_counter() - t0
        self.stats.prompt_tokens += sum(len(s.feed) for s in live)
        t0 = time.perf_counter()
        self._mark = None
        self._steps0 = self.stats.decode_steps
        self._stopwatch()
        try:
            if self.draw is not None:
                self._decode_ahead(live, first, max_new_tokens, stop_ids, include_stop)
            else:
                self._decode(live, first, max_new_tokens, stop_ids, include_stop)
        finally:
            self.sync()
            end = time.perf_counter()
            self.stats.decode_seconds += end - t0
            if self._mark is not None:
                self.stats.timed_seconds += end - self._mark[0]
                self.stats.timed_steps += self.stats.decode_steps - self._mark[1]

    def _stopwatch(self) -> None:
        """Start the stopwatch when the batch has run `time_after` decode steps."""
        if (self.time_after is not None and self._mark is None
                and self.stats.decode_steps - self._steps0 >= self.time_after):
            self.sync()
            self._mark = (time.perf_counter(), self.stats.decode_steps)

    def _read(self, s: _Live, tok: int, stop_ids, include_stop: bool, max_new_tokens: int) -> None:
        """A drawn token has reached the host: count it, keep it, decide whether its sequence ends."""
        s.drawn += 1
        self.stats.generated_tokens += 1
        why = self.ended(tok, s.drawn, s.prompt_len + s.drawn, stop_ids, max_new_tokens,
                         self.max_seq_len)
        if why != "stop" or include_stop:
            s.out.append(tok)
            if self.on_token is not None:
                self.on_token(s.index, tok)
        s.history.append(tok)
        s.why = why

    def _decode_ahead(self, everyone, pending, max_new_tokens, stop_ids, include_stop) -> None:
        """Every decode step is started before the tokens of the step before it have been read."""
        rows = everyone                  # the sequences `pending` has a token for, in order
        while True:
            # who goes on after the pending token unless it is a stop token: known by count
            cont: List[_Live] = []
            places: List[int] = []
            for i, s in enumerate(rows):
                if s.dead:
                    continue
                if self.ended(-1, s.drawn + 1, s.prompt_len + s.drawn + 1, (), max_new_tokens,
                              self.max_seq_len) is None:
                    cont.append(s)
                    places.append(i)
            following = None
            if cont:
                tokens = pending.device if len(places) == len(rows) else pending.pick(places)
                logits = self.step([StepEntry(s.slot, [0], [0]) for s in cont],
                                   device_tokens=tokens)
                following = self.draw(logits, [s.seed for s in cont],
                                      [s.counter0 + s.drawn + 1 for s in cont],
                                      [s.history for s in cont], tokens)
                self.stats.decode_steps += 1
                self._stopwatch()
            for s, tok in zip(rows, pending.tokens()):
                if s.dead:
                    continue             # it drew a stop token a step ago: this one is void
                self._read(s, int(tok), stop_ids, include_stop, max_new_tokens)
                if s.why is not None:
                    s.void_fed = any(s is c for c in cont)   # only a stop token comes unforeseen
                    self._release(s)     # after the step that still used the slot was started
                    s.dead = True
            if following is None:
                break
            rows, pending = cont, following

    def _decode(self, live, tokens, max_new_tokens, stop_ids, include_stop) -> None:
        while True:
            going: List[_Live] = []
            for s, tok in zip(live, tokens):
                self._read(s, int(tok), stop_ids, include_stop, max_new_tokens)
                if s.why is None:
                    going.append(s)
                else:
                    self._release(s)
            live = going
            if not live:
                break
            logits = self.step([StepEntry(s.slot, [s.history[-1]], [0]) for s in live])
            tokens = self.sample(logits, [s.seed for s in live],
                                 [s.counter0 + s.drawn for s in live], [s.history for s in live])
            self.stats.decode_steps += 1
            self._stopwatch()
