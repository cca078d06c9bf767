"""One sequence that goes on over several turns.

The reference's `chat` keeps one context for the whole conversation: every user input is
run on top of what the model has seen (`ModelImp::decode(user_input, token)` executes the new
tokens at `m_past`, src/core/model_imp.cpp:38-52), then tokens are decoded one by one until
the end token (`decode_iter`, :55-65; the loop is application/chat.cpp:221-275), and the token
that ended a turn is never run through the model.  A `Session` does the same with one slot of
the cache: the tokens of a turn are one step that goes on from the slot's length, the answer
is decoded from there, and the slot is given back when the session is closed.
"""
from __future__ import annotations

import time
from typing import Callable, List, Optional, Sequence

import torch

from ..sampling.params import SamplingParams, request_seed
from ..sampling.sampler import Sampler
from .generate import GenerationStats
from .step import StepEntry


class Session:
    """A conversation in one cache slot of an engine (`Engine.session`).

    `say(tokens)` feeds the turn's tokens after everything said so far and returns the tokens
    generated in answer; a token that ended a turn (a stop token) is not fed, as in the
    reference; one that was generated but not yet run when `max_new_tokens` cut the answer is
    fed in front of the next turn.  `remaining`: tokens the context still has room for (the
    reference's `get_remain_token`, src/core/model_imp.h:93)."""

    def __init__(self, engine, params: SamplingParams, stop_token_ids: Optional[Sequence[int]] = None):
        if engine.model.one_token_mixers:
            raise ValueError("a session goes on from the cache by several tokens a turn, which this "
                             "model's " + ", ".join(engine.model.one_token_mixers) + " cannot")
        params.validate()
        self.engine = engine
        self.params = params
        self.sampler = Sampler(params, engine.device)
        self.stops = set(engine.spec.eos_token_ids if stop_token_ids is None else stop_token_ids)
        self.slot: Optional[int] = engine.alloc_slot()
        self.history: List[int] = []          # every token of the conversation, fed or drawn
        self.drawn = 0                        # draws so far (the counter of the next draw)
        self.seed = request_seed(params.seed, 0)
        self._unfed: Optional[int] = None     # drawn and shown, but not run through the model yet
        self.last_stats = GenerationStats()

    # ------------------------------------------------------------ state
    @property
    def length(self) -> int:
        """Tokens the cache holds of this conversation."""
        self._open()
        return self.engine.cache.length(self.slot)

    @property
    def remaining(self) -> int:
        """Tokens that still fit into the context (fed or generated)."""
        return max(0, self.engine.max_seq_len - self.length - (1 if self._unfed is not None else 0))

    def _open(self) -> None:
        if self.slot is None:
            raise ValueError("the session is closed")

    def close(self) -> None:
        if self.slot is not None:
            self.engine.free_slot(self.slot)
            self.slot = None

    def __enter__(self) -> "Session":
        return self

    def __exit__(self, *exc) -> None:
        self.close()

    # ------------------------------------------------------------ a turn
    def _draw(self, logits: torch.Tensor) -> int:
        hist = [self.history] if self.sampler.needs_histories() else None
        token = self.sampler(logits, [self.seed], [self.drawn], hist)[0]
        self.drawn += 1
        self.history.append(token)
        return token

    def say(self, tokens: Sequence[int], max_new_tokens: int = 128,
            on_token: Optional[Callable[[int], None]] = None, include_stop: bool = False) -> List[int]:
        """Feed `tokens` after what was said so far and generate until a stop token, until
        `max_new_tokens` are drawn or until the context is full.  `on_token(token)` is called for
        every token as it comes.  Raises ValueError if the turn does not fit into the context."""
        self._open()
        vocab = self.engine.spec.vocab_size
        turn = [int(t) for t in tokens]
        for t in turn:
            if not 0 <= t < vocab:
                raise ValueError(f"token id {t} outside the vocabulary of {vocab}")
        feed = ([self._unfed] if self._unfed is not None else []) + turn
        if not feed:
            raise ValueError("a turn needs at least one token")
        if len(feed) > self.engine.max_seq_len - self.length:
            raise ValueError(f"the turn's {len(turn)} tokens do not fit: {self.remaining} tokens of "
                             f"the context are left")
        stats = self.last_stats = GenerationStats(prompt_tokens=len(feed), batches=1)
        sync = lambda: torch.cuda.synchronize(self.engine.device)
        out: List[int] = []
        sync()
        start = time.perf_counter()
        # (a step that the cache has no room for raises before it changes anything: the session
        # stays as it was)
        logits = self.engine.step([StepEntry(self.slot, feed, [len(feed) - 1])])
        self.history.extend(turn)
        self._unfed = None
        token = self._draw(logits)
        sync()
        stats.prefill_seconds = time.perf_counter() - start
        start = time.perf_counter()
        while True:
            stop = token in self.stops
            if not stop or include_stop:
                out.append(token)
                stats.generated_tokens += 1
                if on_token is not None:
                    on_token(token)
            if stop:
                break                                   # (the token that ends a turn is not run)
            if len(out) >= max_new_tokens or self.engine.max_seq_len - self.length < 1:
                self._unfed = token                     # shown, to be run with the next turn
                break
            logits = self.engine.step([StepEntry(self.slot, [token], [0])])
            token = self._draw(logits)
            stats.decode_steps += 1
        sync()
        stats.decode_seconds = time.perf_counter() - start
        return out
