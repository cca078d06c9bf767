"""The engine on the GPU against the plain implementation (tests/plain_llama.py),
in float32 and in bfloat16: whole requests, the last 32 tokens one by one, batches
of unequal lengths with slots used again, long decoding, the first tokens of a
sequence, greedy generation through the entry point."""
import math

import pytest
import torch

import plain_llama
from tiny import CONFIGS, make_model_dir, random_ids, read_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# Largest |engine - plain| over a request, divided by the largest |plain logit| of it.
# float32: rounding of sums of a few hundred float32 terms.  bfloat16: activations carry
# 8 bits (2^-8 = 0.4 %) and pass through up to 3 blocks and the head.
BUDGET = {"float32": 2e-5, "bfloat16": 3e-2}
@pytest.mark.parametrize("name,limit", [("A", 1), ("A", 2), ("B", 1), ("A", 5), ("B", 16), ("A", 64)])
def test_generation_with_prompts_fed_in_several_steps(tmp_path_factory, name, limit):
    """`max_step_tokens`: the prompts of a batch in steps of at most that many tokens (sequences
    that go on beside sequences that start); the generated tokens are the plain model's.  A model
    with a mixer that cannot go on by several tokens refuses.  With a limit of 1 every prompt's
    last step is a step of one token that goes on, which is replayed from a decode graph whose
    output the next such step writes again: the logits of a prompt that ended must have been
    taken out by then."""
    config = CONFIGS[name]
    eng, plain, _ = setup(tmp_path_factory, name, "float32", max_batch=3)
    assert eng.runner.use_graphs
    _, w = _cache[(name, "float32")]
    prompts = requests_for(config, [23, 1, 40, 9, 64], seed=12)
    got = eng.generate(prompts, max_new_tokens=5, stop_token_ids=[], max_step_tokens=limit)
    assert got == [plain_llama.generate_greedy(config, w, p, 5) for p in prompts]
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0
    eng.model.one_token_mixers = ["SomeMixer"]            # (what a model with such a mixer reports)
    with pytest.raises(ValueError, match="SomeMixer cannot go on"):
        eng.generate(prompts[:1], max_new_tokens=2, max_step_tokens=4)


STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}

_cache = {}


def setup(tmp_path_factory, name, dtype, **kw):
    """(engine, plain logits function) for a tiny configuration; folders are per session."""
    import inferllm_amd as I
    config = CONFIGS[name]
    key = (name, dtype)
    if key not in _cache:
        d = make_model_dir(tmp_path_factory.getbasetemp(), config, seed=7, dtype=STORE[dtype], gain=4.0)
        _cache[key] = (d, read_weights(d))
    d, w = _cache[key]
    kw.setdefault("max_batch", 4)
    eng = I.Engine.from_pretrained(d, dtype=dtype, device=DEV, poison_freed=True, **kw)
    return eng, (lambda ids: plain_llama.forward_logits(config, w, ids)), config


def err(got, want):
    return float((got.double().cpu() - want).abs().max() / want.abs().max())


def requests_for(config, lens, seed=0):
    return [random_ids(n, config["vocab_size"], seed + 31 * i + n) for i, n in enumerate(lens)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_whole_requests(tmp_path_factory, name, dtype):
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, name, dtype)
    for ids in requests_for(config, [7, 1, 2, 100, 65]):
        s = eng.alloc_slot()
        got = eng.step([StepEntry(s, ids, list(range(len(ids))))])
        assert err(got, plain(ids)) < BUDGET[dtype]
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("copies", [True, False])
def test_short_prompts_at_head_size_128(tmp_path_factory, copies):
    """Prompts of at most 16 tokens take the few-rows kernels in their first step too, where the
    q|k|v product is the plain one: with head size 128 the decode copy of that matrix follows
    other tiles (rows and their rotation partners) and must not be read by it."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "D", "bfloat16", decode_copies=copies)
    for ids in requests_for(config, [1, 5, 16, 17], seed=9):
        s = eng.alloc_slot()
        got = [eng.step([StepEntry(s, ids, list(range(len(ids))))]).clone()]
        more = random_ids(3, config["vocab_size"], 77)
        for t in more:
            got.append(eng.step([StepEntry(s, [t], [0])]).clone())
        assert err(torch.cat(got), plain(ids + more)) < BUDGET["bfloat16"], len(ids)
        eng.free_slot(s)


def test_steps_of_17_to_64_rows(tmp_path_factory, monkeypatch):
    """Steps of 17 to 128 rows (here 24 to 64: a prompt of that length, or that many sequences decoding) read the
    decode copy of the down projection with K cut into ranges, whose planes the next norm adds
    (configuration B: 96 x 256).  24 sequences decode together after prompts of unequal lengths;
    one prompt of 40 tokens runs alone."""
    from inferllm_amd import StepEntry
    from inferllm_amd.kernels import ops
    calls = []
    real = ops.linear_planes
    monkeypatch.setattr(ops, "linear_planes", lambda x, w, *a: calls.append(x.shape[0]) or real(x, w, *a))
    eng, plain, config = setup(tmp_path_factory, "B", "bfloat16", max_batch=24, decode_copies=True)
    ids = requests_for(config, [40], seed=2)[0]
    s = eng.alloc_slot()
    assert err(eng.step([StepEntry(s, ids, list(range(40)))]), plain(ids)) < BUDGET["bfloat16"]
    eng.free_slot(s)
    assert calls and set(calls) == {40}
    del calls[:]
    reqs = requests_for(config, [3 + (5 * i) % 11 for i in range(24)], seed=4)
    heads = [len(r) - 2 for r in reqs]
    slots = [eng.alloc_slot() for _ in reqs]
    got = [[] for _ in reqs]
    out = eng.step([StepEntry(s, r[:h], list(range(h))) for s, r, h in zip(slots, reqs, heads)])
    at = 0
    for i, h in enumerate(heads):
        got[i].append(out[at:at + h].clone())
        at += h
    assert not calls                                     # 139 rows, more than 128: the vendor GEMM
    for t in range(2):
        out = eng.step([StepEntry(s, [r[h + t]], [0]) for s, r, h in zip(slots, reqs, heads)])
        for i in range(len(reqs)):
            got[i].append(out[i:i + 1].clone())
    assert calls and set(calls) <= set(range(24, 65))    # 24 rows, or the bucket they are padded to
    for i, r in enumerate(reqs):
        assert err(torch.cat(got[i]), plain(r)) < BUDGET["bfloat16"], i
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("first", [1, 5, 17])
def test_few_rows_through_the_planes_where_they_pay(tmp_path_factory, monkeypatch, first):
    """From how few rows the down projection goes through planes is a table entry per shape; here it
    is pinned (1: every step; 5: steps of 5 rows or more; 17: never below 17), and prompts of 3
    and 9 tokens and six sequences decoding together must come out as the plain model's in each."""
    from inferllm_amd import StepEntry
    from inferllm_amd.kernels import ops
    # (without graphs: a graph's step has its bucket's rows, and the way is chosen by the rows)
    eng, plain, config = setup(tmp_path_factory, "B", "bfloat16", max_batch=8, decode_copies=True, use_graphs=False)
    shape = (config["hidden_size"], config["intermediate_size"])
    eng.plan.planes_from[shape] = first
    calls = []
    real = ops.linear_planes
    monkeypatch.setattr(ops, "linear_planes", lambda x, w, *a: calls.append(x.shape[0]) or real(x, w, *a))
    for n in (3, 9):
        ids = requests_for(config, [n], seed=n)[0]
        s = eng.alloc_slot()
        assert err(eng.step([StepEntry(s, ids, list(range(n)))]), plain(ids)) < BUDGET["bfloat16"]
        eng.free_slot(s)
    reqs = requests_for(config, [4, 9, 3, 7, 5, 3], seed=8)
    slots = [eng.alloc_slot() for _ in reqs]
    got = [[eng.step([StepEntry(s, r[:-2], list(range(len(r) - 2)))])] for s, r in zip(slots, reqs)]
    for t in (2, 1):
        out = eng.step([StepEntry(s, [r[-t]], [0]) for s, r in zip(slots, reqs)])
        for i in range(len(reqs)):
            got[i].append(out[i:i + 1].clone())
    for i, r in enumerate(reqs):
        assert err(torch.cat(got[i]), plain(r)) < BUDGET["bfloat16"], i
    for s in slots:
        eng.free_slot(s)
    if first == 17:
        assert not calls
    else:
        assert calls and min(calls) >= first and (first > 1 or 1 in calls or 2 in calls)


def test_the_rows_from_which_planes_pay(monkeypatch):
    """By the plan's table; a shape the table lacks follows the rule (from 17 rows) and is timed
    only by a plan that measures, once."""
    from inferllm_amd.kernels import ops
    from inferllm_amd.kernels.plan import Plan
    for shape, measured in (((128, 512), False), ((1024, 4096), True)):
        m = torch.randn(*shape, device="cuda", dtype=torch.bfloat16)
        w = ops.Weight(m, ops.tile_weight(m, ops.tile_rows(shape[0], "plain")), "plain")
        x = torch.zeros(8, shape[1], device="cuda", dtype=torch.bfloat16)
        x17 = torch.zeros(17, shape[1], device="cuda", dtype=torch.bfloat16)
        assert ops.linear_planes_fits(x, w)
        fixed = Plan()
        monkeypatch.setattr(ops, "_plan", fixed)
        assert not ops.linear_planes_pays(x, w) and ops.linear_planes_pays(x17, w)
        assert not fixed.planes_from                       # nothing was timed or remembered
        fixed.planes_from[shape] = 5
        assert ops.linear_planes_pays(x, w) and not ops.linear_planes_pays(x[:4], w)
        tuned = Plan(measure=True)
        monkeypatch.setattr(ops, "_plan", tuned)
        a = ops.linear_planes_pays(x, w)
        first = tuned.planes_from[shape]
        assert first in (1, 5, 9, 13, 17) and (measured or first == 17)    # small ones: never
        assert a == (8 >= first)
        assert ops.linear_planes_pays(x17, w)
        assert Plan.from_dict(tuned.to_dict()) == tuned and not Plan.from_dict(tuned.to_dict()).measure


@pytest.mark.parametrize("copies", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_last_32_tokens_one_by_one(tmp_path_factory, name, dtype, copies):
    """`copies`: with and without the second copy of the matrices that decoding reads."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, name, dtype, decode_copies=copies)
    assert eng.decode_copies == (copies and dtype == "bfloat16")
    for ids in requests_for(config, [33, 100, 128], seed=5):
        want = plain(ids)
        s = eng.alloc_slot()
        head = len(ids) - 32
        got = [eng.step([StepEntry(s, ids[:head], list(range(head)))]).clone()]
        for t in ids[head:]:
            got.append(eng.step([StepEntry(s, [t], [0])]).clone())
        got = torch.cat(got)
        per_pos = (got.double().cpu() - want).abs().max(dim=1).values / want.abs().max()
        assert float(per_pos.max()) < BUDGET[dtype], f"first bad position {int((per_pos >= BUDGET[dtype]).nonzero()[0])}"
        eng.free_slot(s)


@pytest.mark.parametrize("graphs", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_unequal_batches_with_slot_reuse(tmp_path_factory, name, dtype, graphs):
    """Batches of three requests of unequal lengths, one batch after another in two
    slots' worth of spare room; shorter requests end earlier; every position's
    logits equal the plain model's."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, name, dtype, max_batch=3, max_tokens=64 * 5,
                               use_graphs=graphs)
    reqs = requests_for(config, [70, 9, 40, 3, 66, 12, 5, 90, 33], seed=9)
    want = [plain(r) for r in reqs]
    prompt = [max(1, len(r) - 6 - i) for i, r in enumerate(reqs)]
    for b0 in range(0, len(reqs), 3):
        batch = list(range(b0, b0 + 3))
        slot = {i: eng.alloc_slot() for i in batch}
        got = {i: [] for i in batch}
        out = eng.step([StepEntry(slot[i], reqs[i][:prompt[i]], list(range(prompt[i]))) for i in batch])
        o = 0
        for i in batch:
            got[i].append(out[o:o + prompt[i]].clone()); o += prompt[i]
        at = dict((i, prompt[i]) for i in batch)
        live = [i for i in batch if at[i] < len(reqs[i])]
        for i in batch:
            if i not in live:
                eng.free_slot(slot[i])
        while live:
            out = eng.step([StepEntry(slot[i], [reqs[i][at[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                got[i].append(out[j:j + 1].clone()); at[i] += 1
            for i in [i for i in live if at[i] == len(reqs[i])]:
                eng.free_slot(slot[i])
            live = [i for i in live if at[i] < len(reqs[i])]
        for i in batch:
            assert err(torch.cat(got[i]), want[i]) < BUDGET[dtype], f"request {i}"
        eng.cache.check()
        assert eng.cache.slots.n_held() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_a_prompt_cut_into_steps(tmp_path_factory, name, dtype):
    """Attention goes on from the cache by any number of tokens a step: a prompt cut at odd
    places (also across cache pages), a second sequence that starts while the first goes on, a
    step in which one brings many tokens and the other one; every position's logits equal the
    plain model's, whole."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, name, dtype, max_batch=2)
    assert eng.model.one_token_mixers == []
    a, b = requests_for(config, [120, 75], seed=12)
    wa, wb = plain(a), plain(b)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    got_a, got_b = [], []
    got_a.append(eng.step([StepEntry(sa, a[:30], list(range(30)))]).clone())
    got_a.append(eng.step([StepEntry(sa, a[30:31], [0])]).clone())                 # one token: a decode step
    out = eng.step([StepEntry(sa, a[31:100], list(range(69))), StepEntry(sb, b[:70], list(range(70)))])
    got_a.append(out[:69].clone()); got_b.append(out[69:].clone())
    out = eng.step([StepEntry(sb, b[70:71], [0]), StepEntry(sa, a[100:], list(range(20)))])
    got_b.append(out[:1].clone()); got_a.append(out[1:].clone())
    for t in b[71:]:
        got_b.append(eng.step([StepEntry(sb, [t], [0])]).clone())
    for got, want, who in ((got_a, wa, "a"), (got_b, wb, "b")):
        per_pos = (torch.cat(got).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
        assert float(per_pos.max()) < BUDGET[dtype], \
            f"request {who}: first bad position {int((per_pos >= BUDGET[dtype]).nonzero()[0])}"
    eng.free_slot(sa); eng.free_slot(sb)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path_factory, dtype):
    """Decode 250 tokens one by one after a 3-token prompt (crossing several pages)."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "B", dtype)
    ids = requests_for(config, [253], seed=2)[0]
    want = plain(ids)
    s = eng.alloc_slot()
    got = [eng.step([StepEntry(s, ids[:3], [0, 1, 2])]).clone()]
    for t in ids[3:]:
        got.append(eng.step([StepEntry(s, [t], [0])]).clone())
    per_pos = (torch.cat(got).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
    assert float(per_pos.max()) < BUDGET[dtype], f"first bad position {int((per_pos >= BUDGET[dtype]).nonzero()[0])}"
    eng.free_slot(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(tmp_path_factory, dtype):
    """A one-token prompt, then tokens one by one from position 1 on."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "A", dtype)
    ids = requests_for(config, [6], seed=4)[0]
    want = plain(ids)
    s = eng.alloc_slot()
    got = [eng.step([StepEntry(s, [t], [0])]).clone() for t in ids]
    assert err(torch.cat(got), want) < BUDGET[dtype]
    eng.free_slot(s)


def test_padding_and_batch_company_change_nothing_float32(tmp_path_factory):
    """The same request alone and among others: float32 logits agree to rounding."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "B", "float32", max_batch=4)
    reqs = requests_for(config, [40, 7, 19], seed=6)
    s = eng.alloc_slot()
    alone = eng.step([StepEntry(s, reqs[0], [len(reqs[0]) - 1])]).clone()
    eng.free_slot(s)
    slots = [eng.alloc_slot() for _ in reqs]
    out = eng.step([StepEntry(sl, r, [len(r) - 1]) for sl, r in zip(reversed(slots), reqs)])
    assert float((out[0] - alone[0]).abs().max()) < 1e-6
    for sl in slots:
        eng.free_slot(sl)


def test_a_step_takes_its_tokens_from_the_device(tmp_path_factory):
    """`device_tokens`: the tokens of a step of single tokens as an int32 tensor on the device
    (what the sampler left there) instead of the entries' own; the logits are the same bit for
    bit, with and without graphs, and a step of whole prompts refuses them."""
    from inferllm_amd import StepEntry
    from inferllm_amd.engine.step import StepError
    for graphs in (True, False):
        eng, plain, config = setup(tmp_path_factory, "B", "bfloat16", use_graphs=graphs)
        reqs = requests_for(config, [9, 4, 17], seed=6)
        got = {}
        for mode in ("host", "device"):
            slots = [eng.alloc_slot() for _ in reqs]
            eng.step([StepEntry(s, r[:-3], []) for s, r in zip(slots, reqs)])
            rows = []
            for t in range(3):
                toks = [r[len(r) - 3 + t] for r in reqs]
                if mode == "host":
                    out = eng.step([StepEntry(s, [k], [0]) for s, k in zip(slots, toks)])
                else:
                    dev = torch.tensor(toks, dtype=torch.int32, device=DEV)
                    out = eng.step([StepEntry(s, [0], [0]) for s in slots], device_tokens=dev)
                rows.append(out.clone())
            got[mode] = torch.stack(rows)
            for s in slots:
                eng.free_slot(s)
        assert torch.equal(got["host"], got["device"])
        for i, r in enumerate(reqs):
            assert err(got["device"][:, i], plain(r)[-3:]) < BUDGET["bfloat16"]
        s = eng.alloc_slot()
        with pytest.raises(StepError, match="single tokens only"):
            eng.step([StepEntry(s, [1, 2], [1])], device_tokens=torch.zeros(1, dtype=torch.int32, device=DEV))
        eng.step([StepEntry(s, [1, 2], [1])])
        for bad in (torch.zeros(2, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int64, device=DEV),
                    torch.zeros(1, dtype=torch.int32)):
            with pytest.raises(StepError, match="device_tokens"):
                eng.step([StepEntry(s, [3], [0])], device_tokens=bad)
        eng.free_slot(s)
        eng.cache.check()


def test_generation_with_stop_tokens_runs_ahead_and_equals_plain(tmp_path_factory):
    """Greedy requests run one step ahead of the host; a sequence that draws a stop token has one
    void step on its way when the host sees it.  Results and freed slots must be as without."""
    eng, plain, config = setup(tmp_path_factory, "A", "float32", max_batch=3)
    prompts = requests_for(config, [5, 11, 2, 7, 3], seed=2)
    want = [plain_llama.generate_greedy(config, _cache[("A", "float32")][1], p, 12) for p in prompts]
    stops = {want[0][3], want[2][0], want[3][7]}
    cut = []
    for w in want:
        k = next((i for i, t in enumerate(w) if t in stops), len(w))
        cut.append(w[:k])
    assert eng.generate(prompts, max_new_tokens=12, stop_token_ids=sorted(stops)) == cut
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_equals_plain(tmp_path_factory, name):
    import inferllm_amd as I
    config = CONFIGS[name]
    eng, plain, _ = setup(tmp_path_factory, name, "float32", max_batch=2)
    _, w = _cache[(name, "float32")]
    prompts = requests_for(config, [7, 11, 2, 5, 30], seed=8)
    n_new = 9 if name == "A" else 6
    got = eng.generate(prompts, max_new_tokens=n_new, stop_token_ids=[])
    want = [plain_llama.generate_greedy(config, w, p, n_new) for p in prompts]
    assert got == want
    # a stop token ends its sequence early and is left out
    stop = want[1][2]
    got = eng.generate(prompts[:3], max_new_tokens=n_new, stop_token_ids=[stop])
    assert got == [plain_llama.generate_greedy(config, w, p, n_new, [stop]) for p in prompts[:3]]
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0


def test_sampling_with_a_repeat_penalty_is_the_same_step_by_step_and_running_ahead(tmp_path_factory):
    """The repeat penalty's window ends with the newest token, which the loop that runs ahead has
    only on the device: both loops must draw the same tokens."""
    import inferllm_amd as I
    from inferllm_amd.engine import GenerationLoop
    from inferllm_amd.sampling import Sampler, SamplingParams
    eng, plain, config = setup(tmp_path_factory, "B", "float32", max_batch=3)
    prompts = requests_for(config, [5, 11, 2, 9], seed=8)
    params = SamplingParams(temperature=0.9, top_k=20, top_p=0.9, repeat_penalty=1.4, repeat_last_n=5, seed=3)
    outs = []
    for ahead in (False, True):
        sampler = Sampler(params, DEV)
        loop = GenerationLoop(eng.step, sampler, eng.alloc_slot, eng.free_slot, max_batch=3,
                              max_tokens=eng.cache.max_tokens, max_seq_len=eng.max_seq_len,
                              draw=sampler.draw if ahead else None)
        outs.append(loop.run(prompts, params, 10, [7, 9, 11]))
        eng.cache.check()
    assert outs[0] == outs[1] and any(len(o) > 3 for o in outs[0])
    strong = eng.generate(prompts, temperature=0.9, top_k=20, top_p=0.9, repeat_penalty=1.4, repeat_last_n=5,
                          seed=3, max_new_tokens=10, stop_token_ids=[7, 9, 11])
    assert strong == outs[0]
    none = eng.generate(prompts, temperature=0.9, top_k=20, top_p=0.9, seed=3, max_new_tokens=10,
                        stop_token_ids=[7, 9, 11])
    assert none != strong                                  # the penalty does change the draws


def test_temperature_sampling_is_reproducible_and_batch_independent(tmp_path_factory):
    eng, plain, config = setup(tmp_path_factory, "B", "float32", max_batch=3)
    prompts = requests_for(config, [5, 11, 2], seed=1)
    a = eng.generate(prompts, temperature=0.8, seed=42, max_new_tokens=6, stop_token_ids=[])
    b = eng.generate(prompts, temperature=0.8, seed=42, max_new_tokens=6, stop_token_ids=[])
    c = eng.generate(prompts, temperature=0.8, seed=43, max_new_tokens=6, stop_token_ids=[])
    assert a == b and a != c
    eng1, _, _ = setup(tmp_path_factory, "B", "float32", max_batch=1)     # one at a time
    assert eng1.generate(prompts, temperature=0.8, seed=42, max_new_tokens=6, stop_token_ids=[]) == a


def test_command_line_generates_like_the_plain_model(tmp_path):
    """`bin/chat` with token-id prompts, greedy: the same tokens as the plain implementation."""
    import os
    import subprocess
    import sys
    config = CONFIGS["A"]
    d = make_model_dir(tmp_path, config, seed=7, dtype=torch.float32, gain=4.0)
    w = read_weights(d)
    prompts = requests_for(config, [7, 3], seed=3)
    ids_file = tmp_path / "prompts.txt"
    ids_file.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "chat"), "-m", d, "-d", "float32", "--temp", "0",
                        "-n", "9", "--prompt-ids-file", str(ids_file), "-c", "64", "--summary", "--type", "llama2"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    got = [[int(t) for t in line.split()] for line in r.stdout.strip().splitlines()]
    want = [plain_llama.generate_greedy(config, w, p, 9, [2]) for p in prompts]
    assert got == want
    assert "token/s" in r.stderr
    bad = subprocess.run([sys.executable, os.path.join(root, "bin", "chat"), "-m", d, "--type", "chatglm",
                          "--prompt-ids", "1 2"], capture_output=True, text=True, timeout=110)
    assert bad.returncode == 2 and "does not fit" in bad.stderr


def test_a_session_keeps_one_context_over_its_turns(tmp_path):
    """`Engine.session`: turns fed one after another into one slot give the tokens that the plain
    model gives for the whole conversation; an answer cut by `max_new_tokens` leaves its last
    token to be fed with the next turn, a stop token ends a turn and is never fed; the context's
    end and the slot's return are kept track of."""
    import inferllm_amd as I
    config = CONFIGS["A"]
    d = make_model_dir(tmp_path, config, seed=17, dtype=torch.float32, gain=4.0)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="float32", device=DEV, max_batch=2, max_seq_len=48, poison_freed=True)
    turns = requests_for(config, [9, 4, 3], seed=6)
    seen = []
    with eng.session(stop_token_ids=[]) as talk:
        said = list(turns[0])
        a1 = talk.say(turns[0], max_new_tokens=5, on_token=seen.append)
        assert a1 == plain_llama.generate_greedy(config, w, said, 5) and seen == a1
        assert talk.length == len(said) + 4 and talk.remaining == 48 - len(said) - 5     # the fifth is not fed yet
        said += a1 + list(turns[1])
        a2 = talk.say(turns[1], max_new_tokens=3)
        assert a2 == plain_llama.generate_greedy(config, w, said, 3)
        said += a2
        assert talk.last_stats.prompt_tokens == 1 + len(turns[1]) and talk.last_stats.generated_tokens == 3
        with pytest.raises(ValueError, match="do not fit"):
            talk.say([1] * 40)
        assert talk.length == len(said) - 1                        # nothing was fed by the refused turn
        slot = talk.slot
    assert talk.slot is None
    both = [eng.alloc_slot(), eng.alloc_slot()]                     # the slot is free again
    assert slot in both
    for s_ in both:
        eng.free_slot(s_)
    eng.cache.check()
    with pytest.raises(ValueError, match="closed"):
        talk.say([1])
    # a stop token: a token of the first answer that none before it equals ends the turn; it is
    # not returned and not fed
    j = next(j for j in range(1, 5) if a1[j] not in a1[:j])
    stop = a1[j]
    with eng.session(stop_token_ids=[stop]) as talk:
        b1 = talk.say(turns[0], max_new_tokens=5)
        assert b1 == a1[:j] and talk.length == len(turns[0]) + j
        said = list(turns[0]) + b1 + list(turns[2])
        b2 = talk.say(turns[2], max_new_tokens=4, include_stop=True)
        want = plain_llama.generate_greedy(config, w, said, 4, [stop])
        assert b2[:len(want)] == want and (len(want) == 4 or b2[len(want)] == stop)
    # the context's end: generation stops when nothing more fits, the rest of the answer is cut
    with eng.session(stop_token_ids=[]) as talk:
        out = talk.say(requests_for(config, [40], seed=8)[0], max_new_tokens=100)
        assert len(out) == 9 and talk.length == 48 and talk.remaining == 0     # the ninth cannot be fed any more
    eng.cache.check()
    # no pages left for a turn: the error leaves the session as it was, and the turn goes
    # through once another session has given its pages back
    from inferllm_amd.cache import CacheFull
    eng = I.Engine.from_pretrained(d, dtype="float32", device=DEV, max_batch=2, max_tokens=128, poison_freed=True)
    first, second = eng.session(stop_token_ids=[]), eng.session(stop_token_ids=[])
    first.say(requests_for(config, [70], seed=3)[0], max_new_tokens=2)       # both pages
    with pytest.raises(CacheFull):
        second.say(turns[0], max_new_tokens=5)
    assert second.length == 0 and second.history == [] and second.remaining == eng.max_seq_len
    first.close()
    assert second.say(turns[0], max_new_tokens=5) == a1
    second.close()
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0


def test_command_line_turns_from_standard_input_share_one_context(tmp_path):
    """`bin/chat` without a prompt: the lines of standard input are turns of one conversation,
    as in the reference's loop."""
    import os
    import subprocess
    import sys
    config = CONFIGS["A"]
    d = make_model_dir(tmp_path, config, seed=7, dtype=torch.float32, gain=4.0)
    w = read_weights(d)
    turns = requests_for(config, [6, 3], seed=5)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "chat"), "-m", d, "-d", "float32", "--temp", "0",
                        "-n", "4", "-c", "64", "--stop-ids", "100000"],
                       input="\n".join(" ".join(map(str, t)) for t in turns) + "\n",
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stderr
    got = [[int(t) for t in line.split()] for line in r.stdout.strip().splitlines()]
    first = plain_llama.generate_greedy(config, w, turns[0], 4)
    second = plain_llama.generate_greedy(config, w, list(turns[0]) + first + list(turns[1]), 4)
    assert got == [first, second]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompt_then_decoding_at_head_size_128(tmp_path_factory, dtype):
    """1,500 tokens in one step (many query blocks, key tiles and pages), then 40 tokens one by
    one at positions beyond 1,500, with the head size and grouping of the large models."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "D", dtype, max_batch=2, max_seq_len=2048,
                               max_tokens=2048 + 64)
    ids = requests_for(config, [1540], seed=12)[0]
    want = plain(ids)
    s = eng.alloc_slot()
    probe = [0, 1, 63, 64, 127, 128, 129, 700, 1023, 1024, 1499]
    got = eng.step([StepEntry(s, ids[:1500], probe)]).clone()
    per = (got.double().cpu() - want[probe]).abs().max(dim=1).values / want.abs().max()
    assert float(per.max()) < BUDGET[dtype], f"prefill rows {[p for p, e in zip(probe, per) if e >= BUDGET[dtype]]}"
    outs = [eng.step([StepEntry(s, [t], [0])]).clone() for t in ids[1500:]]
    per = (torch.cat(outs).double().cpu() - want[1500:]).abs().max(dim=1).values / want.abs().max()
    assert float(per.max()) < BUDGET[dtype], f"first bad decode position {1500 + int((per >= BUDGET[dtype]).nonzero()[0])}"
    eng.free_slot(s)
    eng.cache.check()


def test_a_context_beyond_4096_beside_a_short_one(tmp_path_factory):
    """A prompt of 4,300 tokens and one of 70 in one step, then six tokens each: the long
    sequence's keys lie in the class of lengths up to 8,192, the most splits, and rotation
    angles at positions that a table of 4,096 would not hold."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "E", "bfloat16", max_batch=2, max_seq_len=8192,
                               max_tokens=4480 + 128)
    reqs = requests_for(config, [4306, 76], seed=3)
    wants = [plain(r) for r in reqs]
    slots = [eng.alloc_slot() for _ in reqs]
    probes = [[0, 63, 64, 2047, 2048, 4095, 4096, 4299], [0, 69]]
    got = eng.step([StepEntry(s, r[:-6], p) for s, r, p in zip(slots, reqs, probes)])
    at = 0
    for w, p in zip(wants, probes):
        assert err(got[at:at + len(p)], w[p]) < BUDGET["bfloat16"]
        at += len(p)
    for t in range(6, 0, -1):
        out = eng.step([StepEntry(s, [r[-t]], [0]) for s, r in zip(slots, reqs)])
        for i, (w, r) in enumerate(zip(wants, reqs)):
            assert err(out[i:i + 1], w[len(r) - t:len(r) - t + 1]) < BUDGET["bfloat16"], (i, t)
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_batch_of_a_hundred_sequences(tmp_path_factory, dtype):
    """More sequences than any few-rows kernel takes (100: a decode bucket of 128 rows, products
    by the vendor GEMM in bfloat16): prompts of unequal lengths in one step, then three tokens
    each; every sequence is compared with the plain implementation."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "B", dtype, max_batch=100, max_seq_len=64)
    reqs = requests_for(config, [4 + (7 * i) % 13 for i in range(100)], seed=40)
    heads = [len(r) - 3 for r in reqs]
    slots = [eng.alloc_slot() for _ in reqs]
    out = eng.step([StepEntry(s, r[:h], [h - 1]) for s, r, h in zip(slots, reqs, heads)])
    got = [[out[i:i + 1].clone()] for i in range(100)]
    for t in range(3):
        out = eng.step([StepEntry(s, [r[h + t]], [0]) for s, r, h in zip(slots, reqs, heads)])
        for i in range(100):
            got[i].append(out[i:i + 1].clone())
    worst = 0.0
    for i, (r, h) in enumerate(zip(reqs, heads)):
        want = plain(r)[h - 1:]
        worst = max(worst, err(torch.cat(got[i]), want))
    assert worst < BUDGET[dtype]
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


def test_decode_copies_of_the_thin_matrices_alone(tmp_path_factory):
    """`decode_copies="thin"` (what the engine chooses when copies of all matrices do not fit):
    only the down projections, which have K >= 2 N, get the second copy."""
    from inferllm_amd import StepEntry
    from inferllm_amd.kernels import ops
    eng, plain, config = setup(tmp_path_factory, "B", "bfloat16", decode_copies="thin", max_batch=24)
    assert eng.decode_copies == "thin"
    for layer in eng.model.layers:
        assert isinstance(layer.feed_forward.w_down, ops.Weight) and layer.feed_forward.w_down.mode == "plain"
        assert not isinstance(layer.feed_forward.w_gate_up, ops.Weight)
        assert not isinstance(layer.mixer.w_qkv, ops.Weight) and not isinstance(layer.mixer.w_o, ops.Weight)
    for n in (1, 9, 40):                                  # few-rows kernels, and the split product
        ids = requests_for(config, [n + 3], seed=30 + n)[0]
        s = eng.alloc_slot()
        got = [eng.step([StepEntry(s, ids[:n], list(range(n)))]).clone()]
        for t in ids[n:]:
            got.append(eng.step([StepEntry(s, [t], [0])]).clone())
        assert err(torch.cat(got), plain(ids)) < BUDGET["bfloat16"], n
        eng.free_slot(s)


def test_decoding_across_a_class_of_lengths(tmp_path_factory):
    """Decode graphs are captured per class of lengths (up to 1024 keys, 2048, ...), since how
    attention cuts the keys among blocks is fixed at capture: two sequences decode from 1,010
    and 1,020 keys to beyond 1,024, through the change of graph."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "D", "bfloat16", max_batch=2, max_seq_len=2048,
                               max_tokens=2 * 1088)
    reqs = requests_for(config, [1040, 1050], seed=21)
    heads = [1010, 1020]
    slots = [eng.alloc_slot() for _ in reqs]
    eng.step([StepEntry(s, r[:h], []) for s, r, h in zip(slots, reqs, heads)])
    got = [[], []]
    for t in range(30):
        out = eng.step([StepEntry(s, [r[h + t]], [0]) for s, r, h in zip(slots, reqs, heads)])
        got[0].append(out[0:1].clone()); got[1].append(out[1:2].clone())
    assert len(eng.runner._graphs) == 2 and {k[1] for k in eng.runner._graphs} == {1024, 2048}
    for i, (r, h) in enumerate(zip(reqs, heads)):
        want = plain(r[:h + 30])[h:h + 30]
        per = (torch.cat(got[i]).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
        assert float(per.max()) < BUDGET["bfloat16"], f"request {i}: first bad position {h + int((per >= BUDGET['bfloat16']).nonzero()[0])}"
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("graphs", [True, False])
def test_decoding_sequences_of_widely_different_lengths(tmp_path_factory, graphs):
    """A decode step whose sequences differ widely in length (the longest 1,024 keys or more, the
    mean at most 0.6 of it) has its keys cut into more ranges, and graphs of its own: sequences
    of 1,100, 40 and 200 keys side by side, until the short ones end and the long one alone is
    no longer such a step."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "D", "bfloat16", max_batch=3, max_seq_len=2048,
                               max_tokens=1152 + 64 + 256, use_graphs=graphs)
    heads = [1100, 40, 200]
    tails = [12, 5, 8]
    reqs = requests_for(config, [h + t for h, t in zip(heads, tails)], seed=27)
    slots = [eng.alloc_slot() for _ in reqs]
    eng.step([StepEntry(s, r[:h], []) for s, r, h in zip(slots, reqs, heads)])
    got = [[] for _ in reqs]
    for t in range(max(tails)):
        live = [i for i in range(3) if t < tails[i]]
        out = eng.step([StepEntry(slots[i], [reqs[i][heads[i] + t]], [0]) for i in live])
        for row, i in enumerate(live):
            got[i].append(out[row:row + 1].clone())
    if graphs:       # three and two sequences in the graph of 4 and of 2 rows, the last one alone
        assert set(eng.runner._graphs) == {(4, 2048, True), (2, 2048, True), (1, 2048, False)}
    for i, r in enumerate(reqs):
        want = plain(r)[heads[i]:]
        per = (torch.cat(got[i]).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
        assert float(per.max()) < BUDGET["bfloat16"], (i, per.tolist())
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


def test_kernel_timing_reports_every_op(tmp_path_factory):
    from inferllm_amd.kernels.profile import kernel_timing
    eng, plain, config = setup(tmp_path_factory, "A", "bfloat16", use_graphs=False)
    with kernel_timing() as t:
        out = eng.generate([[1, 2, 3, 4]], max_new_tokens=3, stop_token_ids=[])
    tot = t.totals()
    assert len(out[0]) == 3
    for op in ("embed", "add_rmsnorm", "linear", "attn_prefill", "attn_decode", "argmax"):
        assert tot[op][0] > 0 and tot[op][1] > 0.0, op
    # every norm of the prompt's step is a launch; single-token steps take the norm inside the
    # product that follows wherever the sizes allow, the last norm always remains
    n_norms = 2 * config["num_hidden_layers"] + 1
    assert n_norms + 2 <= tot["add_rmsnorm"][0] <= 3 * n_norms
    assert "share" in t.table()


def test_warm_up_captures_the_decode_graphs_beforehand(tmp_path):
    """`Engine.warm_up` captures the graphs of the batch sizes named (their buckets, once each)
    without touching a sequence, and runs a throwaway prompt if asked to: the steps that follow
    capture nothing more and give the same bits as in an engine that was not warmed up; an engine
    without graphs has nothing to do."""
    import inferllm_amd as I
    from inferllm_amd import StepEntry
    config = CONFIGS["B"]
    d = make_model_dir(tmp_path, config, seed=31, dtype=torch.bfloat16, gain=4.0)
    reqs = requests_for(config, [9, 14, 5, 11, 7], seed=4)

    def run(warm):
        eng = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=8, poison_freed=True)
        if warm:
            assert eng.warm_up([1, 5, 6, 8], longest=40) == 2           # graphs of 1 and of 8 rows
            assert eng.warm_up([5], prompt_tokens=70) == 0             # there already; a throwaway prompt
            assert eng.cache.slots.n_held() == 0                       # whose slot and pages came back
            eng.cache.check()
            before = dict(eng.runner._graphs)
        slots = [eng.alloc_slot() for _ in reqs]
        eng.step([StepEntry(s, r[:-3], []) for s, r in zip(slots, reqs)])
        outs = [eng.step([StepEntry(s, [r[len(r) - 3 + t]], [0]) for s, r in zip(slots, reqs)]).clone()
                for t in range(3)]
        if warm:
            assert eng.runner._graphs.keys() == before.keys()
        return outs

    cold, warm = run(False), run(True)
    for a, b in zip(cold, warm):
        assert torch.equal(a, b)
    eager = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=8, use_graphs=False)
    assert eager.warm_up() == 0


def test_head_size_80_in_bfloat16(tmp_path_factory):
    """A LLaMA of width 2560 with 32 heads of 80 (grouped in fours), a head size that is no
    multiple of 32: the matrix-core prompt kernel with its last block of dims half used, the
    fused q|k|v product with rotation, decode attention, whole prompts (one longer than a block
    of 128 query rows) and single tokens, 3 and then 20 sequences together."""
    import inferllm_amd as I
    from inferllm_amd import StepEntry
    config = {"architectures": ["LlamaForCausalLM"], "hidden_size": 2560, "intermediate_size": 6912,
              "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8,
              "vocab_size": 4000, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
              "max_position_embeddings": 512, "tie_word_embeddings": False,
              "bos_token_id": 1, "eos_token_id": 2}
    d = make_model_dir(tmp_path_factory.getbasetemp(), config, seed=13, dtype=torch.bfloat16, gain=2.0)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=20, max_seq_len=256,
                                   poison_freed=True)
    assert eng.spec.layers[0].mixer.params["head_dim"] == 80
    tail = 4
    reqs = requests_for(config, [170, 23, 70] + [6 + i % 5 for i in range(17)], seed=7)
    heads = [len(r) - tail for r in reqs]
    slots = [eng.alloc_slot() for _ in reqs]
    out = eng.step([StepEntry(s, r[:h], list(range(h)) if i < 3 else []) for i, (s, r, h) in enumerate(zip(slots, reqs, heads))])
    got = {i: [] for i in range(len(reqs))}
    at = 0
    for i in range(3):
        got[i].append(out[at:at + heads[i]].clone())
        at += heads[i]
    for t in range(tail):
        live = range(3) if t < 2 else range(len(reqs))
        if t == 2:                                       # the short ones catch up, then all 20 go on together
            for u in range(2):
                eng.step([StepEntry(slots[i], [reqs[i][heads[i] + u]], []) for i in range(3, len(reqs))])
        out = eng.step([StepEntry(slots[i], [reqs[i][heads[i] + t]], [0]) for i in live])
        for row, i in enumerate(live):
            got[i].append(out[row:row + 1].clone())
    for i in (0, 1, 2, 5, 19):
        want = plain_llama.forward_logits(config, w, reqs[i])
        want = want[:len(reqs[i])] if i < 3 else want[heads[i] + 2:heads[i] + tail]
        per_pos = (torch.cat(got[i]).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
        assert float(per_pos.max()) < BUDGET["bfloat16"], \
            f"request {i}: first bad position {int((per_pos >= BUDGET['bfloat16']).nonzero()[0])} of {len(per_pos)}"
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


@pytest.mark.parametrize("n,later,buckets", [(40, 25, [32, 48]), (70, 55, [64, 96])])
@pytest.mark.parametrize("nkv,ffn", [(32, 11008), (8, 14336)])
def test_real_layer_sizes_with_many_sequences(tmp_path_factory, monkeypatch, nkv, ffn, n, later, buckets):
    """Two layers of the LLaMA-2-7B sizes (and of the LLaMA-3-8B ones: heads grouped in fours, a
    q|k|v matrix of 6144 rows) with 40, then 25 sequences decoding together (and with 70, then
    55): steps of 17 to 128 rows take the kernels that share X through LDS (fused q|k|v with
    rotation and store, gate|up with SiLU-multiply, o and down as planes, the head) from graphs
    of 48 and of 32 rows (of 96 and of 64), and no product of such a step goes to the vendor
    GEMM."""
    import inferllm_amd as I
    from inferllm_amd import StepEntry
    config = {"architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "intermediate_size": ffn,
              "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": nkv,
              "vocab_size": 32000, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
              "max_position_embeddings": 512, "tie_word_embeddings": False,
              "bos_token_id": 1, "eos_token_id": 2}
    d = make_model_dir(tmp_path_factory.getbasetemp() / f"many{nkv}", config, seed=12, dtype=torch.bfloat16, gain=2.0)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=n, max_seq_len=64,
                                   poison_freed=True)
    assert eng.decode_copies is True
    tail = 5
    reqs = requests_for(config, [5 + (3 * i) % 6 + tail for i in range(n)], seed=5)
    heads = [len(r) - tail for r in reqs]
    slots = [eng.alloc_slot() for _ in reqs]
    eng.step([StepEntry(s, r[:h], []) for s, r, h in zip(slots, reqs, heads)])
    vendor = []
    real = torch.matmul
    monkeypatch.setattr(torch, "matmul", lambda *a, **k: vendor.append(tuple(a[0].shape)) or real(*a, **k))
    live = list(range(n))
    got = {i: [] for i in live}
    for t in range(tail):
        if t == 3:                                       # 15 sequences end: the rest goes on in a smaller graph
            for i in live[later:]:
                eng.free_slot(slots[i])
            live = live[:later]
        out = eng.step([StepEntry(slots[i], [reqs[i][heads[i] + t]], [0]) for i in live])
        for row, i in enumerate(live):
            got[i].append(out[row:row + 1].clone())
    monkeypatch.setattr(torch, "matmul", real)
    assert not vendor, f"products of decode steps went to the vendor GEMM: rows x width {sorted(set(vendor))}"
    assert sorted(k[0] for k in eng.runner._graphs) == buckets
    for i in sorted({0, 7, 16, later - 1, later, n - 7, n - 1}):   # the plain model is slow at these sizes
        want = plain_llama.forward_logits(config, w, reqs[i])[heads[i]:heads[i] + len(got[i])]
        per_pos = (torch.cat(got[i]).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
        assert float(per_pos.max()) < BUDGET["bfloat16"], f"request {i}: {per_pos.tolist()}"
    for i in live:
        eng.free_slot(slots[i])
    eng.cache.check()


@pytest.mark.parametrize("nkv,ffn", [(32, 11008), (8, 14336)])
def test_real_layer_sizes_in_bfloat16(tmp_path_factory, nkv, ffn):
    """Two layers of the LLaMA-2-7B sizes (width 4096, 32 heads of 128, feed-forward 11008,
    vocabulary 32000) and of the LLaMA-3-8B ones (8 kv heads, feed-forward 14336): the sizes
    the serving kernels are tuned for, which the tiny configurations never reach (products
    over 4096 and 11008, 256 parts of a row's sum of squares, the vendor GEMM and the
    matrix-core attention for the prompt, grouped decode attention on the matrix cores)."""
    import inferllm_amd as I
    from inferllm_amd import StepEntry
    config = {"architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "intermediate_size": ffn,
              "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": nkv,
              "vocab_size": 32000, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
              "max_position_embeddings": 512, "tie_word_embeddings": False,
              "bos_token_id": 1, "eos_token_id": 2}
    d = make_model_dir(tmp_path_factory.getbasetemp(), config, seed=11, dtype=torch.bfloat16, gain=2.0)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=4, poison_freed=True)
    reqs = requests_for(config, [40, 23, 70], seed=3)
    heads = [len(r) - 6 for r in reqs]
    slots = [eng.alloc_slot() for _ in reqs]
    got = [[] for _ in reqs]
    out = eng.step([StepEntry(s, r[:h], list(range(h))) for s, r, h in zip(slots, reqs, heads)])
    at = 0
    for i, h in enumerate(heads):
        got[i].append(out[at:at + h].clone())
        at += h
    for t in range(6):                                   # three rows: a padded bucket of four
        out = eng.step([StepEntry(s, [r[h + t]], [0]) for s, r, h in zip(slots, reqs, heads)])
        for i in range(len(reqs)):
            got[i].append(out[i:i + 1].clone())
    for i, r in enumerate(reqs):
        want = plain_llama.forward_logits(config, w, r)
        per_pos = (torch.cat(got[i]).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
        assert float(per_pos.max()) < BUDGET["bfloat16"], \
            f"request {i}: first bad position {int((per_pos >= BUDGET['bfloat16']).nonzero()[0])} of {len(r)}"
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()


def near_best(want_rows, tokens, budget):
    """Whether each generated token is one whose plain logit lies within twice `budget` (of the
    largest plain logit) of the row's best: what greedy decoding may pick when the engine's
    logits are within `budget` of the plain ones."""
    top = float(want_rows.abs().max())
    return all(float(row.max() - row[t]) <= 2 * budget * top for row, t in zip(want_rows, tokens))


@pytest.mark.parametrize("limit", [1, 7, 40])
def test_prompts_fed_in_several_steps_in_bfloat16(tmp_path_factory, limit):
    """`max_step_tokens` in bfloat16, with graphs on: every generated token is near the best of
    the plain model's logits along the sequence the engine produced, and the engine's own logits
    over that sequence, fed whole, are within the budget."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, "B", "bfloat16", max_batch=3)
    prompts = requests_for(config, [23, 2, 40, 9, 64], seed=14)
    got = eng.generate(prompts, max_new_tokens=6, stop_token_ids=[], max_step_tokens=limit)
    whole = setup(tmp_path_factory, "B", "bfloat16", max_batch=3)[0].generate(
        prompts, max_new_tokens=6, stop_token_ids=[])
    for p, g, g0 in zip(prompts, got, whole):
        assert len(g) == 6
        want = plain(list(p) + g)
        assert near_best(want[len(p) - 1:len(p) + 5], g, BUDGET["bfloat16"]), (limit, len(p))
        # the first token comes from the same rows of the same kernels' classes as without the
        # limit only in rounding: where they differ, both are near the best
        if g != g0:
            assert near_best(plain(list(p) + g0)[len(p) - 1:len(p) + 5], g0, BUDGET["bfloat16"])
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_session_decodes_through_graphs_across_a_class_of_lengths(tmp_path_factory, dtype):
    """A conversation whose answer grows from 1,000 to beyond 1,024 keys: the loop behind
    `Session.say` runs ahead through decode graphs of a batch of one, and changes to the graph of
    the next class of lengths on the way.  A second turn goes on from there."""
    eng, plain, config = setup(tmp_path_factory, "D", dtype, max_batch=2, max_seq_len=2048,
                               max_tokens=2 * 1152)
    first, second = requests_for(config, [1000, 30], seed=23)
    with eng.session(stop_token_ids=[]) as talk:
        a1 = talk.say(first, max_new_tokens=40)
        assert len(a1) == 40 and talk.length == 1039
        a2 = talk.say(second, max_new_tokens=8)
        assert talk.last_stats.prompt_tokens == 31 and talk.length == 1039 + 31 + 7
    assert {k for k in eng.runner._graphs} == {(1, 1024, False), (1, 2048, False)}
    seq = list(first) + a1 + list(second) + a2
    want = plain(seq)
    if dtype == "float32":
        assert a1 == [int(t) for t in want[999:1039].argmax(dim=1)]
        assert a2 == [int(t) for t in want[1069:1077].argmax(dim=1)]
    else:
        assert near_best(want[999:1039], a1, BUDGET[dtype]) and near_best(want[1069:1077], a2, BUDGET[dtype])
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0


def test_a_session_whose_answer_breaks_off_for_want_of_pages(tmp_path):
    """The page pool is shared: when an answer finds no page for its next token the step raises,
    and the session stands where the last step that ran left it: the tokens shown so far are the
    conversation (the exception carries them), and the next turn goes on behind them once there
    is room."""
    import inferllm_amd as I
    from inferllm_amd.cache import CacheFull
    config = CONFIGS["A"]
    d = make_model_dir(tmp_path, config, seed=17, dtype=torch.float32, gain=4.0)
    w = read_weights(d)
    for graphs in (True, False):
        eng = I.Engine.from_pretrained(d, dtype="float32", device=DEV, max_batch=2, max_tokens=128,
                                       poison_freed=True, use_graphs=graphs)
        a, b = eng.session(stop_token_ids=[]), eng.session(stop_token_ids=[])
        turn = requests_for(config, [60, 5, 3], seed=40)
        a.say(turn[1], max_new_tokens=2)                       # a holds one of the two pages
        shown = []
        with pytest.raises(CacheFull) as caught:
            b.say(turn[0], max_new_tokens=20, on_token=shown.append)   # 60 + 20 tokens need a second page
        want = plain_llama.generate_greedy(config, w, turn[0], 8)
        # the sequence can hold 64 tokens: 60 of the turn and four of the answer were run
        assert b.length == 64 and shown == want[:len(shown)] and len(shown) in (4, 5)
        assert caught.value.generated == shown
        assert b.history == list(turn[0]) + shown
        a.close()
        said = list(turn[0]) + shown + list(turn[2])
        assert b.say(turn[2], max_new_tokens=3) == plain_llama.generate_greedy(config, w, said, 3)
        b.close()
        eng.cache.check()
        assert eng.cache.slots.n_held() == 0


def depth_budget(layers: int) -> float:
    """The bfloat16 budget as a function of depth: a block rounds the activations between its
    kernels to 8 bits (2^-9 relative, on average) at half a dozen places, and what the blocks add
    to the float32 residual stream is independent from block to block, so the error of the
    logits, as a fraction of the largest, grows like the square root of the number of blocks.
    1.5 % for one block and the head is what the tiny models' budget of 3 % allows their three
    blocks."""
    return 1.5e-2 * math.sqrt(layers + 1)


@pytest.mark.parametrize("layers", [8, 32])
def test_bfloat16_error_grows_with_the_square_root_of_depth(tmp_path_factory, layers):
    """Width 2,048 (16 heads of 128 on 4 kv heads, feed-forward 5,632, vocabulary 3,001), 8 and 32
    layers: a prompt whole, then tokens one by one, against the plain model on the same rounded
    matrices.  No tiny model shows what depth does to bfloat16.  (Measured with these weights at
    2, 4, 8 and 16 layers: 0.46, 0.55, 0.53 and 0.55 of the budget, so the square root holds.)"""
    import inferllm_amd as I
    from inferllm_amd import StepEntry
    config = {"architectures": ["LlamaForCausalLM"], "hidden_size": 2048, "intermediate_size": 5632,
              "num_hidden_layers": layers, "num_attention_heads": 16, "num_key_value_heads": 4,
              "vocab_size": 3001, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
              "max_position_embeddings": 256, "tie_word_embeddings": False,
              "bos_token_id": 1, "eos_token_id": 2}
    d = make_model_dir(tmp_path_factory.getbasetemp() / f"deep{layers}", config, seed=31, dtype=torch.bfloat16,
                       gain=1.5)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=2, poison_freed=True)
    ids = requests_for(config, [28], seed=9)[0]
    want = plain_llama.forward_logits(config, w, ids)
    s = eng.alloc_slot()
    got = [eng.step([StepEntry(s, ids[:20], list(range(20)))])]
    for t in ids[20:]:
        got.append(eng.step([StepEntry(s, [t], [0])]))
    eng.free_slot(s)
    per_pos = (torch.cat(got).double().cpu() - want).abs().max(dim=1).values / want.abs().max()
    assert float(per_pos.max()) < depth_budget(layers), per_pos.tolist()
    # and the budget is no empty promise: the error is of the budget's order, not far below it
    assert float(per_pos.max()) > depth_budget(layers) / 30


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_short_prompt_steps_are_replayed_from_graphs(tmp_path_factory, name, dtype):
    """Steps of several tokens a sequence with few rows (short prompts, a conversation's turns)
    run eagerly the first time a shape comes and from a HIP graph from the second time on: rows
    that only fill the graph up are a sequence of their own on the spare slot, sequences that
    only fill it up are empty.  Whole prompts, ragged batches, steps that go on from the cache,
    wanted rows anywhere; and the cache they leave serves the decode steps that follow."""
    from inferllm_amd import StepEntry
    eng, plain, config = setup(tmp_path_factory, name, dtype, max_batch=6)
    assert eng.runner.use_graphs
    budget = BUDGET[dtype]
    for round_ in range(3):                                  # eager, capture + replay, replay
        for batch in ([9], [3, 30, 1], [40, 41, 17, 70, 2]):
            reqs = requests_for(config, [n + 4 for n in batch], seed=50 + 7 * round_ + len(batch))
            slots = [eng.alloc_slot() for _ in reqs]
            want = [plain(r) for r in reqs]
            # the prompts but their last four tokens, logits wanted at the first and the last row
            out = eng.step([StepEntry(s, r[:n], [0, n - 1] if n > 1 else [0]) for s, r, n in zip(slots, reqs, batch)])
            at = 0
            for i, n in enumerate(batch):
                for p_ in ([0, n - 1] if n > 1 else [0]):
                    assert err(out[at], want[i][p_]) < budget, (round_, batch, i, p_)
                    at += 1
            assert at == out.shape[0]
            # two more tokens in a step that goes on from the cache (rows over the paged cache)
            out = eng.step([StepEntry(s, r[n:n + 2], [1]) for s, r, n in zip(slots, reqs, batch)])
            for i, n in enumerate(batch):
                assert err(out[i], want[i][n + 1]) < budget, (round_, batch, i)
            # and single tokens: the cache holds what the graphs' steps stored
            for t in (2, 3):
                out = eng.step([StepEntry(s, [r[n + t]], [0]) for s, r, n in zip(slots, reqs, batch)])
                for i, n in enumerate(batch):
                    assert err(out[i], want[i][n + t]) < budget, (round_, batch, i, t)
            for s in slots:
                eng.free_slot(s)
            eng.cache.check()
    keys = set(eng.runner._prompt_graphs)
    # (rows, sequences, goes on): 9 and 2 rows in 16, 34 and 6 in 64 and 16, 170 and 10 in 192 and 16
    assert keys == {(16, 2, False), (16, 2, True), (64, 4, False), (16, 4, True), (192, 8, False), (16, 8, True)}
    assert all(g.graph is not None for g in eng.runner._prompt_graphs.values())
    # more rows or more wanted rows than a graph holds, and a step that wants nothing: eagerly
    s = eng.alloc_slot()
    ids = requests_for(config, [60], seed=77)[0]
    before = dict(eng.runner._prompt_uses)
    out = eng.step([StepEntry(s, ids, list(range(60)))])
    assert err(out, plain(ids)) < budget and eng.runner._prompt_uses == before
    eng.free_slot(s)
