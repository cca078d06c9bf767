"""One sequence that goes on over several turns.

The reference's `chat` keeps one context for the whole conversation: every user input is
run on top of what the model has seen (`ModelImp::decode(user_input, token)` executes the new
tokens at `m_past`, src/core/model_imp.cpp:38-52), then tokens are decoded one by one until
the end token (`decode_iter`, :55-65; the loop is application/chat.cpp:221-275), and the token
that ended a turn is never run through the model.  A `Session` does the same with one slot of
the cache: the tokens of a turn are one step that goes on from the slot's length, the answer
is decoded from there, and the slot is given back when the session is closed.  The decoding is
the generation loop's, with a batch of one in a slot that the session owns, so a conversation
runs one step ahead of the host like any other batch.
"""
from __future__ import annotations

from typing import Callable, List, Optional, Sequence

from ..sampling.params import SamplingParams, request_seed
from ..sampling.sampler import Sampler
from .generate import GenerationStats


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
    def say(self, tokens: Sequence[int], max_new_tokens: int = 128,
            on_token: Optional[Callable[[int], None]] = None, include_stop: bool = False) -> List[int]:
        """Feed `tokens` after what was said so far and generate until a stop token, until
        `max_new_tokens` are drawn or until the context is full.  `on_token(token)` is called for
        every token as it comes.  Raises ValueError if the turn does not fit into the context.

        A step that the cache has no room for raises (`CacheFull`; the page pool is shared with
        other sessions and batches).  The session then stands where the last step that ran left
        it: a turn whose first step found no room has not happened; an answer that broke off
        keeps the tokens shown so far (the exception carries them as `generated`), and the next
        turn goes on behind them."""
        self._open()
        engine = self.engine
        vocab = engine.spec.vocab_size
        turn = [int(t) for t in tokens]
        for t in turn:
            if not 0 <= t < vocab:
                raise ValueError(f"token id {t} outside the vocabulary of {vocab}")
        feed = ([self._unfed] if self._unfed is not None else []) + turn
        if not feed:
            raise ValueError("a turn needs at least one token")
        held = self.length
        if len(feed) > engine.max_seq_len - held:
            raise ValueError(f"the turn's {len(turn)} tokens do not fit: {self.remaining} tokens of "
                             f"the context are left")
        # a void step (the one the loop has started when a stop token turns up) can be taken back
        # from keys and values, not from a mixer's own state: such a model is decoded in step
        loop = engine.generation_loop(self.sampler, ahead=not engine.cache.states,
                                      on_token=(lambda _i, tok: on_token(tok)) if on_token else None)
        self.last_stats = loop.stats
        history = self.history + turn
        record = None
        try:
            record = loop.run_turn(self.slot, held, feed, history, self.seed, self.drawn,
                                   max_new_tokens, self.stops, include_stop)
        except Exception as e:
            now = engine.cache.length(self.slot)
            if now == held:
                raise                                   # the turn's first step did not run
            if now < held + len(feed):
                self.close()                            # a part of the turn ran: nothing to go on from
                raise
            # the turn ran and `history` holds every token that was read since; all of them
            # were run except, when the loop decodes in step, the newest
            answer = history[len(self.history) + len(turn):]
            self._settle(history, held + len(feed), len(answer))
            self.history = history
            e.generated = list(answer)
            raise
        self._settle(history, held + len(feed), record.drawn)
        self.history = history
        if record.why == "stop":
            self._unfed = None                          # the token that ends a turn is never run
        return record.out

    def _settle(self, history: List[int], fed_len: int, drawn: int) -> None:
        """After a turn (or what ran of it): count the draws and find the token that was shown
        but not run, from what the cache holds."""
        self.drawn += drawn
        missing = fed_len + drawn - self.engine.cache.length(self.slot)
        self._unfed = history[-1] if drawn > 0 and missing >= 1 else None
