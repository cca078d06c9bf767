"""The generation loop's decisions, with a fake model in place of the GPU:
batches, stop tokens, sequences that end earlier, limits, slots given back."""
import pytest

from inferllm_amd.engine import GenerationLoop, StepEntry, plan_prefill
from inferllm_amd.sampling import SamplingParams, request_seed, uniform


class FakeModel:
    """next token = (sum of the sequence so far) % 50; keeps its own view of each slot."""

    def __init__(self, n_slots, takes_cut_prompts=False):
        self.free = list(range(n_slots - 1, -1, -1))
        self.seq = {}
        self.steps = []
        self.max_live = 0
        self.takes_cut_prompts = takes_cut_prompts     # steps that go on by several tokens

    def alloc(self):
        s = self.free.pop()
        self.seq[s] = []
        return s

    def release(self, s):
        assert s in self.seq, "slot freed twice"
        del self.seq[s]
        self.free.append(s)

    def step(self, entries, device_tokens=None):
        first = [len(self.seq[e.slot]) == 0 for e in entries]
        assert (self.takes_cut_prompts or all(first)
                or (not any(first) and all(len(e.tokens) == 1 for e in entries)))
        if device_tokens is not None:
            assert not any(first) and len(device_tokens) == len(entries)
        for i, e in enumerate(entries):
            self.seq[e.slot].extend(e.tokens if device_tokens is None else [device_tokens[i]])
        self.steps.append([(e.slot, len(e.tokens)) for e in entries])
        self.max_live = max(self.max_live, len(self.seq))
        # a row for every wanted place, which is the entry's last token if any
        assert all(list(e.want) in ([], [len(e.tokens) - 1]) for e in entries)
        rows = [sum(self.seq[e.slot]) % 50 for e in entries if list(e.want)]
        return rows or None

    @staticmethod
    def sample(logits, seeds, counters, histories):
        return list(logits)

    @staticmethod
    def draw(logits, seeds, counters, histories, latest=None):
        return FakeDraw(list(logits))


class FakeDraw:
    """What a sampler's `draw` returns: the tokens "on the device", some of them, and on the host."""

    def __init__(self, tokens):
        self.device = tokens

    def pick(self, rows):
        return [self.device[i] for i in rows]

    def tokens(self):
        return list(self.device)


def expected(prompt, n, stops=(), include_stop=False, limit=10**9):
    seq, out = list(prompt), []
    for _ in range(n):
        t = sum(seq) % 50
        if t in stops:
            if include_stop:
                out.append(t)
            break
        out.append(t)
        seq.append(t)
        if len(seq) > limit:      # the token could not be fed back
            break
    return out


def loop_for(model, max_batch=3, max_tokens=64 * 12, max_seq_len=256, ahead=False):
    """ahead: with a `draw`, so that the loop starts every step before it has read the last
    step's tokens."""
    return GenerationLoop(model.step, model.sample, model.alloc, model.release, max_batch,
                          max_tokens, max_seq_len, draw=model.draw if ahead else None)


AHEAD = pytest.mark.parametrize("ahead", [False, True])


PROMPTS = [[1, 2, 3], [7], [4, 4, 4, 4, 9], [10, 11], [3, 3], [8, 1, 1, 1, 1, 1, 2], [5]]


@AHEAD
def test_every_request_gets_its_own_continuation_in_batches_of_three(ahead):
    m = FakeModel(3)
    loop = loop_for(m, ahead=ahead)
    out = loop.run(PROMPTS, SamplingParams(), 6)
    assert out == [expected(p, 6) for p in PROMPTS]
    assert m.max_live <= 3 and not m.seq                    # slots all given back
    assert loop.stats.batches == 3 and loop.stats.prompt_tokens == sum(map(len, PROMPTS))
    # first step of each batch carries whole prompts, later ones single tokens
    assert m.steps[0] == [(0, 3), (1, 1), (2, 5)]
    assert all(n == 1 for s in m.steps[1:6] for _, n in s)


@AHEAD
def test_stop_tokens_end_a_sequence_early_and_the_rest_goes_on(ahead):
    stops = {expected(PROMPTS[0], 6)[2], expected(PROMPTS[2], 6)[0]}
    m = FakeModel(3)
    out = loop_for(m, ahead=ahead).run(PROMPTS[:3], SamplingParams(), 6, stops)
    assert out == [expected(p, 6, stops) for p in PROMPTS[:3]]
    assert out[2] == [] and len(out[0]) == 2 and len(out[1]) > 2
    sizes = [len(s) for s in m.steps]
    if ahead:       # a stop token is seen one step late: that sequence has one void step more
        assert sizes[:3] == [3, 3, 2] and sizes[-1] == 1
        assert len(m.steps) <= 6                         # ends by max_new_tokens are known beforehand: no void step
    else:
        assert sizes[0] == 3 and sizes[1] == 2 and sizes[-1] == 1   # the batch shrinks
    assert not m.seq
    out = loop_for(FakeModel(3), ahead=ahead).run(PROMPTS[:3], SamplingParams(), 6, stops, include_stop=True)
    assert out == [expected(p, 6, stops, True) for p in PROMPTS[:3]]


@AHEAD
def test_context_limit_ends_a_sequence(ahead):
    m = FakeModel(2)
    out = loop_for(m, max_batch=2, max_seq_len=6, ahead=ahead).run([[1, 2, 3], [9, 9, 9, 9, 9, 9]], SamplingParams(), 10)
    assert max(len(v) for v in m.seq.values()) <= 6 if m.seq else True
    assert all(n <= 1 for st in m.steps[1:] for _, n in st)
    assert out == [expected([1, 2, 3], 10, limit=6), expected([9] * 6, 10, limit=6)]
    assert len(out[0]) == 4 and len(out[1]) == 1
    with pytest.raises(ValueError, match="longer than"):
        loop_for(FakeModel(2), max_seq_len=6).run([[1] * 7], SamplingParams(), 1)
    with pytest.raises(ValueError, match="empty prompt"):
        loop_for(FakeModel(2)).run([[]], SamplingParams(), 1)


def test_batches_respect_cache_room():
    loop = loop_for(FakeModel(8), max_batch=8, max_tokens=64 * 4)
    lens = [60, 10, 70, 5, 5]
    assert loop.room_needed(60, 6) == 128 and loop.room_needed(10, 6) == 64
    assert loop.next_batch([0, 1, 2, 3, 4], lens, 6) == [0, 1]           # 128 + 64, then 128 does not fit
    assert loop.next_batch([2, 3, 4], lens, 6) == [2, 3, 4]
    big = loop_for(FakeModel(8), max_batch=8, max_tokens=64 * 4, max_seq_len=2048)
    with pytest.raises(ValueError, match="more cache room"):
        big.next_batch([0], [1000], 6)
    for ahead in (False, True):
        m = FakeModel(8)
        loop = loop_for(m, max_batch=8, max_tokens=64 * 4, ahead=ahead)
        prompts = [[1] * n for n in lens]
        assert loop.run(prompts, SamplingParams(), 6) == [expected(p, 6) for p in prompts]
        assert loop.stats.batches == 2


def test_zero_new_tokens_and_slots_returned_on_error():
    m = FakeModel(2)
    assert loop_for(m).run(PROMPTS[:2], SamplingParams(), 0) == [[], []]

    def broken(entries):
        raise RuntimeError("boom")
    for draw in (None, m.draw):
        loop = GenerationLoop(broken, m.sample, m.alloc, m.release, 2, 640, 64, draw=draw)
        with pytest.raises(RuntimeError, match="boom"):
            loop.run(PROMPTS[:2], SamplingParams(), 3)
        assert not m.seq and len(m.free) == 2


def test_draws_depend_on_request_and_count_only():
    calls = []

    def sample(logits, seeds, counters, histories):
        calls.append((list(seeds), list(counters)))
        return list(logits)
    m = FakeModel(3)
    GenerationLoop(m.step, sample, m.alloc, m.release, 2, 6400, 64).run(PROMPTS[:3], SamplingParams(seed=9), 3)
    assert calls[0] == ([request_seed(9, 0), request_seed(9, 1)], [0, 0])
    assert calls[1][1] == [1, 1] and calls[3] == ([request_seed(9, 2)], [0])
    us = [uniform(request_seed(9, i), c) for i in range(3) for c in range(50)]
    assert all(0.0 <= u < 1.0 for u in us) and len(set(us)) == len(us)
    assert abs(sum(us) / len(us) - 0.5) < 0.1


def test_sampling_params_validation():
    SamplingParams(temperature=0.8, top_k=40, top_p=0.95, repeat_penalty=1.1).validate()
    for bad in (dict(temperature=-1), dict(top_p=0.0), dict(top_p=1.5), dict(repeat_penalty=0),
                dict(repeat_last_n=1000)):
        with pytest.raises(ValueError):
            SamplingParams(**bad).validate()
    assert SamplingParams().greedy and not SamplingParams(temperature=0.1).greedy


@AHEAD
def test_tokens_are_reported_as_they_are_kept(ahead):
    seen = []
    m = FakeModel(3)
    loop = GenerationLoop(m.step, m.sample, m.alloc, m.release, 3, 6400, 256,
                          on_token=lambda i, t: seen.append((i, t)), draw=m.draw if ahead else None)
    stops = {expected(PROMPTS[0], 6)[2]}
    out = loop.run(PROMPTS[:3], SamplingParams(), 4, stops)
    for i in range(3):
        assert [t for j, t in seen if j == i] == out[i]
    assert [i for i, _ in seen[:3]] == [0, 1, 2]          # step by step, not request by request


def test_running_ahead_gives_every_draw_the_same_window_of_earlier_tokens():
    """A draw that looks back (the repeat penalty) sees the same tokens either way: when the loop
    runs ahead, the newest one comes as `latest` (unread) and the ones before it as history."""
    seen = {False: [], True: []}
    m = None

    def sample(logits, seeds, counters, histories):
        seen[False].append([tuple(h) for h in histories])
        return m.sample(logits, seeds, counters, histories)

    def draw(logits, seeds, counters, histories, latest=None):
        whole = [tuple(h) + ((latest[i],) if latest is not None else ()) for i, h in enumerate(histories)]
        seen[True].append(whole)
        return m.draw(logits, seeds, counters, histories)
    outs = []
    for ahead in (False, True):
        m = FakeModel(3)
        loop = GenerationLoop(m.step, sample, m.alloc, m.release, 3, 6400, 256, draw=draw if ahead else None)
        outs.append(loop.run(PROMPTS[:3], SamplingParams(temperature=0.5, repeat_penalty=1.1), 5))
    assert outs[0] == outs[1]
    assert seen[False] == seen[True]


def test_random_stops_and_limits_give_the_same_with_and_without_running_ahead():
    import random
    rng = random.Random(5)
    for trial in range(60):
        prompts = [[rng.randrange(50) for _ in range(rng.randrange(1, 9))] for _ in range(rng.randrange(1, 8))]
        stops = set(rng.sample(range(50), rng.randrange(0, 12)))
        n_new = rng.randrange(1, 9)
        limit = rng.choice([8, 10, 256])
        include = rng.random() < 0.5
        got = []
        for ahead in (False, True):
            m = FakeModel(3)
            loop = loop_for(m, max_seq_len=limit, ahead=ahead)
            got.append(loop.run(prompts, SamplingParams(), n_new, stops, include))
            assert not m.seq and len(m.free) == 3
        assert got[0] == got[1] == [expected(p, n_new, stops, include, limit) for p in prompts], trial


def test_plan_of_prompts_cut_into_steps():
    assert plan_prefill([5, 3], 100) == [[(0, 0, 5), (1, 0, 3)]]
    # the rest of the prompt under way first, then the next ones while there is room
    assert plan_prefill([10, 3, 4], 6) == [[(0, 0, 6)], [(0, 6, 4), (1, 0, 2)], [(1, 2, 1), (2, 0, 4)]]
    assert plan_prefill([2, 2, 2], 4) == [[(0, 0, 2), (1, 0, 2)], [(2, 0, 2)]]
    assert plan_prefill([3], 1) == [[(0, 0, 1)], [(0, 1, 1)], [(0, 2, 1)]]
    for lens, limit in (([7, 1, 30, 2], 8), ([64, 64], 64), ([1, 1, 1], 2)):
        steps = plan_prefill(lens, limit)
        assert all(0 < sum(n for _, _, n in st) <= limit for st in steps)
        fed = [0] * len(lens)
        for st in steps:
            for i, start, n in st:
                assert start == fed[i]                      # every prompt in order, nothing twice
                fed[i] += n
        assert fed == lens
        assert sum(1 for st in steps if sum(n for _, _, n in st) < limit) <= 1    # only the last step is not full
    with pytest.raises(ValueError, match="at least 1"):
        plan_prefill([3], 0)


@AHEAD
@pytest.mark.parametrize("limit", [1, 4, 6, 100])
def test_prompts_fed_in_several_steps_give_the_same_tokens(ahead, limit):
    m = FakeModel(3, takes_cut_prompts=True)
    loop = GenerationLoop(m.step, m.sample, m.alloc, m.release, 3, 64 * 12, 256,
                          draw=m.draw if ahead else None, max_step_tokens=limit)
    out = loop.run(PROMPTS, SamplingParams(), 5)
    assert out == [expected(p, 5) for p in PROMPTS]
    assert not m.seq and loop.stats.prompt_tokens == sum(map(len, PROMPTS))
    # no step of prompts holds more tokens than the limit (single-token steps of the batch aside)
    assert all(sum(n for _, n in st) <= max(limit, 3) for st in m.steps)
    if limit == 4:
        # the first batch's prompts of 3, 1 and 5 tokens: [3 + 1], [4 of the third], [its last]
        assert m.steps[:3] == [[(0, 3), (1, 1)], [(2, 4)], [(2, 1)]]


def test_rows_of_the_decode_graphs():
    """A decode step of n sequences is replayed from a graph of at least n rows: powers of two,
    and from 24 on the sizes half way between them; never fewer rows than sequences, and from 17
    sequences on less than half as many again."""
    from inferllm_amd.engine.step import _bucket
    assert [_bucket(n) for n in (1, 2, 3, 8, 9, 16, 17, 24, 25, 33, 48, 49, 65, 96, 97, 129, 193)] == \
           [1, 2, 4, 8, 16, 16, 24, 24, 32, 48, 48, 64, 96, 96, 128, 192, 256]
    for n in range(1, 600):
        b = _bucket(n)
        assert n <= b and (b < 2 * n or n == 1) and (n < 17 or 2 * b < 3 * n)
        assert b == _bucket(b)


def test_steps_whose_lengths_differ_widely_get_more_key_ranges_within_bounds():
    """The step function calls a decode step ragged when its longest sequence has 1,024 keys or
    more and the mean length is at most 0.6 of that; attention then doubles the key ranges of
    every sequence while there are fewer than 8, as long as that makes no more than 1,024 blocks, and never cuts
    into fewer ranges than for even lengths."""
    from inferllm_amd.engine.step import _ragged
    from inferllm_amd.kernels.ops import decode_splits
    assert _ragged([1101, 41, 201]) and _ragged([4000] + [200] * 15)
    assert not _ragged([1101]) and not _ragged([1000, 10]) and not _ragged([2000, 1900, 1500])
    assert not _ragged([1024, 1024 * 6 // 10 + 1]) and _ragged([1030, 200])
    for nh, nkv in ((32, 32), (32, 8), (64, 8), (4, 2), (7, 7)):
        blocks_a_range = nkv * -(-(nh // nkv) // 16) if nh > nkv else nkv
        for B in (1, 2, 3, 4, 8, 16, 24, 32, 64, 128, 256):
            for longest in (1024, 2048, 4096, 32768):
                even, waves = decode_splits(B, nkv, longest, nh, 128)
                more, waves_r = decode_splits(B, nkv, longest, nh, 128, ragged=True)
                assert more >= even and more in (even, 2 * even, 4 * even, 8 * even) and waves_r in (4, 8)
                if more > even:
                    assert more < 16 and B * blocks_a_range * more <= 1024      # doubled only from fewer than 8
                elif even < 8:
                    assert B * blocks_a_range * even * 2 > 1024
            # short sequences are left alone: a range is at least a tile of keys anyway
            assert decode_splits(B, nkv, 640, nh, 128, ragged=True) == decode_splits(B, nkv, 640, nh, 128)
    assert decode_splits(16, 8, 3800, 32, 128, ragged=True) == (8, 4)
    assert decode_splits(64, 32, 2000, 32, 128, ragged=True) == decode_splits(64, 32, 2000, 32, 128) == (1, 4)


def test_command_line_text_through_a_sentencepiece_model(tmp_path, capsys):
    """`bin/chat -p` takes text through the folder's tokenizer.json or, without one, through its
    tokenizer.model (SentencePiece, as LLaMA-2 checkpoints bring it): a small model trained here
    encodes and decodes a sentence, BOS in front as the reference puts it (model_imp.cpp:123-125);
    a folder with neither refuses text with a clear message."""
    spm = pytest.importorskip("sentencepiece")
    from inferllm_amd.cli.chat import _Text
    corpus = tmp_path / "corpus.txt"
    corpus.write_text("\n".join(["the quick brown fox jumps over the lazy dog",
                                 "a model of language reads tokens and writes tokens",
                                 "one two three four five six seven eight nine ten"] * 20))
    folder = tmp_path / "model"
    folder.mkdir()
    spm.SentencePieceTrainer.train(input=str(corpus), model_prefix=str(folder / "tokenizer"), vocab_size=60,
                                   model_type="bpe", minloglevel=2)
    text = _Text(str(folder))
    ids = text.encode("the quick fox", bos=1)
    assert ids[0] == 1 and len(ids) > 1 and all(isinstance(i, int) and 0 <= i < 60 for i in ids)
    assert text.show(ids[1:]) == "the quick fox"
    put = text.printer()                                   # an answer printed as its tokens come
    capsys.readouterr()
    for t in ids[1:]:
        put(t)
    assert capsys.readouterr().out == "the quick fox"
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(SystemExit, match="tokenizer"):
        _Text(str(empty)).encode("x", bos=None)
    assert _Text(str(empty)).show([3, 4]) == "3 4"
    put = _Text(str(empty)).printer()
    put(3); put(4)
    assert capsys.readouterr().out == "3 4 "


class TurnModel(FakeModel):
    """A fake model whose slots the caller owns, with `rewind`."""

    def rewind(self, slot, n):
        assert 0 < n <= len(self.seq[slot])
        del self.seq[slot][-n:]
        self.rewound = getattr(self, "rewound", 0) + n


@AHEAD
def test_a_turn_in_a_slot_that_the_caller_owns(ahead):
    """`run_turn`: one sequence goes on, in a slot that is not given back, from what it holds;
    the loop leaves in it everything that was run.  A stop token is never run: when the loop
    runs ahead its void step is taken back from the slot."""
    m = TurnModel(2, takes_cut_prompts=True)
    loop = GenerationLoop(m.step, m.sample, m.alloc, m.release, 2, 6400, 256, draw=m.draw if ahead else None,
                          rewind_slot=m.rewind)
    slot = m.alloc()
    first = [4, 4, 9]
    history = list(first)
    r = loop.run_turn(slot, 0, first, history, seed=1, draws_before=0, max_new_tokens=4)
    want = expected(first, 4)
    assert r.out == want and r.why == "length" and history == first + want
    assert m.seq[slot] == first + want[:3]                   # the last drawn token is still to be run
    # the next turn brings that token in front of its own; a stop token ends it
    turn = [want[3], 7, 1]
    said = first + want + [7, 1]
    ans = expected(said, 6)
    stop = ans[2]
    history += [7, 1]
    r = loop.run_turn(slot, len(m.seq[slot]), turn, history, seed=1, draws_before=4, max_new_tokens=6,
                      stop_token_ids=[stop])
    j = ans.index(stop)
    assert r.out == ans[:j] and r.why == "stop" and r.drawn == j + 1
    assert m.seq[slot] == said + ans[:j]                    # the stop token is not in the slot
    assert getattr(m, "rewound", 0) == (1 if ahead else 0)
    assert slot in m.seq and len(m.free) == 1               # the slot is still the caller's
    assert loop.stats.prompt_tokens == 6 and loop.stats.batches == 2    # the loop's stats add up over its calls
    with pytest.raises(ValueError, match="at least one token"):
        loop.run_turn(slot, len(m.seq[slot]), [], history, 1, 0, 3)
    if ahead:
        with pytest.raises(ValueError, match="rewind_slot"):
            GenerationLoop(m.step, m.sample, m.alloc, m.release, 2, 6400, 256, draw=m.draw).run_turn(
                slot, len(m.seq[slot]), [1], history, 1, 0, 3)


def test_a_turn_counts_draws_and_lengths_from_what_the_slot_holds():
    """The sampler's counter goes on from the draws before, and the context's end is counted
    with the tokens the slot held before the turn."""
    calls = []

    def draw(logits, seeds, counters, histories, latest=None):
        calls.append(list(counters))
        return FakeDraw(list(logits))
    m = TurnModel(1, takes_cut_prompts=True)
    loop = GenerationLoop(m.step, m.sample, m.alloc, m.release, 1, 6400, max_seq_len=10, draw=draw,
                          rewind_slot=m.rewind)
    slot = m.alloc()
    m.seq[slot] = [1, 2, 3, 4, 5, 6]
    history = [1, 2, 3, 4, 5, 6, 7, 8]
    r = loop.run_turn(slot, 6, [7, 8], history, seed=0, draws_before=11, max_new_tokens=50)
    assert calls[0] == [11] and calls[1] == [12]
    assert r.why == "context" and len(m.seq[slot]) == 10 and len(r.out) == 3   # the third cannot be run any more
    assert r.out == expected([1, 2, 3, 4, 5, 6, 7, 8], 50, limit=10)


def test_logits_of_a_prompt_that_ended_are_taken_out_at_once():
    """A step's logits may be memory that the next step writes again (a decode graph's output):
    when prompts are fed in several steps, the loop keeps a prompt's last-token row through
    `keep` before the next step runs."""
    buffer = [None]                                          # the one place every step writes to

    class Reusing(FakeModel):
        def step(self, entries, device_tokens=None):
            rows = super().step(entries, device_tokens)
            if rows is None:
                return None
            buffer[0] = list(rows)
            return buffer                                    # a view: logits[0] is the live list

    m = Reusing(3, takes_cut_prompts=True)
    loop = GenerationLoop(m.step, lambda lg, *a: [row[0] if isinstance(row, list) else row for row in lg],
                          m.alloc, m.release, 3, 6400, 256, max_step_tokens=1,
                          keep=lambda logits, row: list(logits[0])[row], join=list)
    prompts = [[1, 2, 3], [7, 5], [4, 4]]
    out = loop.run(prompts, SamplingParams(), 1)
    assert out == [expected(p, 1) for p in prompts]
