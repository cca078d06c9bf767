"""The step function, the cache and the model wiring on the CPU, with the GPU
kernels replaced by their plain torch contracts (tests/kernel_refs.py).  What is
tested here is bookkeeping: packing, positions, page tables, slot reuse, which
rows get logits.  The kernels themselves are tested on the GPU."""
import json
import os

import pytest
import torch

import kernel_refs
import plain_llama
from tiny import CONFIGS, make_model_dir, random_ids, read_weights

import inferllm_amd as I
from inferllm_amd.cache import CacheManager
from inferllm_amd.engine import DecoderModel, StepEntry, StepError, StepRunner


def build_runner(config, weights, max_tokens=1024, max_slots=4, dtype=torch.float32, poison=True):
    cfg = I.config_from_dict(config)
    model = DecoderModel(cfg.to_spec())
    model.load({k: v.to(dtype) if v.is_floating_point() else v for k, v in weights.items()})
    cache = CacheManager(model.kv_lines(), model.state_lines(), max_tokens=max_tokens,
                         max_slots=max_slots, max_seq_len=cfg.max_position_embeddings,
                         dtype=dtype, device="cpu", poison_freed=poison)
    return StepRunner(model, cache, dtype, torch.device("cpu"), use_graphs=False)


@pytest.fixture
def emulated(monkeypatch):
    kernel_refs.patch(monkeypatch)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompt_equals_plain(name, tmp_path, emulated):
    config = CONFIGS[name]
    d = make_model_dir(tmp_path, config, seed=3, gain=4.0)
    w = read_weights(d)
    ids = random_ids(70, config["vocab_size"], 1)
    want = plain_llama.forward_logits(config, w, ids)
    r = build_runner(config, w)
    s = r.cache.alloc_slot()
    got = r.step([StepEntry(s, ids, list(range(len(ids))))])
    assert got.shape == want.shape and got.dtype == torch.float32
    assert (got.double() - want).abs().max() < 1e-5
    r.cache.free_slot(s)
    r.cache.check()


def test_tail_decoding_and_ragged_batches_equal_plain(tmp_path, emulated):
    config = CONFIGS["B"]
    d = make_model_dir(tmp_path, config, seed=5, gain=4.0)
    w = read_weights(d)
    V = config["vocab_size"]
    reqs = [random_ids(n, V, 10 + n) for n in (70, 9, 131, 66, 3)]
    plain = [plain_llama.forward_logits(config, w, ids) for ids in reqs]
    r = build_runner(config, w, max_tokens=64 * 6, max_slots=2)
    # each alone: all but the last 5 tokens whole, then one by one
    for ids, want in zip(reqs, plain):
        s = r.cache.alloc_slot()
        head = max(1, len(ids) - 5)
        got = [r.step([StepEntry(s, ids[:head], list(range(head)))])]
        for t in ids[head:]:
            got.append(r.step([StepEntry(s, [t], [0])]))
        got = torch.cat(got)
        assert (got.double() - want).abs().max() < 1e-5
        r.cache.free_slot(s)
    # batches of two with unequal lengths; the shorter one ends earlier; slots are used again
    for a, b in ((0, 1), (2, 3), (4, 0)):
        sa, sb = r.cache.alloc_slot(), r.cache.alloc_slot()
        pa, pb = max(1, len(reqs[a]) - 4), max(1, len(reqs[b]) - 2)
        out = r.step([StepEntry(sa, reqs[a][:pa], [pa - 1]), StepEntry(sb, reqs[b][:pb], [0, pb - 1])])
        assert (out[0].double() - plain[a][pa - 1]).abs().max() < 1e-5
        assert (out[1].double() - plain[b][0]).abs().max() < 1e-5
        assert (out[2].double() - plain[b][pb - 1]).abs().max() < 1e-5
        ia, ib = pa, pb
        while ia < len(reqs[a]) or ib < len(reqs[b]):
            entries, expect = [], []
            if ia < len(reqs[a]):
                entries.append(StepEntry(sa, [reqs[a][ia]], [0])); expect.append(plain[a][ia]); ia += 1
            if ib < len(reqs[b]):
                entries.append(StepEntry(sb, [reqs[b][ib]], [0])); expect.append(plain[b][ib]); ib += 1
                if ib == len(reqs[b]):
                    pass
            out = r.step(entries)
            for o, e in zip(out, expect):
                assert (o.double() - e).abs().max() < 1e-5
            if ib == len(reqs[b]) and sb is not None:
                r.cache.free_slot(sb); sb = None
        r.cache.free_slot(sa)
        if sb is not None:
            r.cache.free_slot(sb)
        r.cache.check()
    assert r.cache.slots.n_held() == 0 and all(g.pool.n_held() == 0 for g in r.cache.groups)


def test_step_refuses_mixed_phases_and_bad_ids(tmp_path, emulated):
    config = CONFIGS["A"]
    w = read_weights(make_model_dir(tmp_path, config, seed=1, gain=4.0))
    r = build_runner(config, w)
    a, b = r.cache.alloc_slot(), r.cache.alloc_slot()
    r.step([StepEntry(a, [1, 2, 3], [])])
    # a model with a mixer that cannot go on by several tokens (attention with a window, a mixer
    # that does not say it can) takes steps that all start or all go on by one token only
    assert r.model.one_token_mixers == []
    r.model.one_token_mixers = ["SomeMixer"]
    with pytest.raises(StepError, match="all start.*SomeMixer"):
        r.step([StepEntry(a, [4], [0]), StepEntry(b, [1, 2], [1])])
    with pytest.raises(StepError, match="all start"):
        r.step([StepEntry(a, [4, 5], [0])])
    assert r.cache.length(a) == 3 and r.cache.length(b) == 0          # refused before anything was reserved
    r.model.one_token_mixers = []
    with pytest.raises(StepError, match="vocabulary"):
        r.step([StepEntry(a, [256], [0])])
    with pytest.raises(StepError, match="wanted place"):
        r.step([StepEntry(a, [5], [1])])
    with pytest.raises(StepError, match="twice"):
        r.step([StepEntry(a, [5], [0]), StepEntry(a, [6], [0])])
    assert r.step([StepEntry(a, [5], [])]) is None



def test_a_prompt_cut_into_steps_equals_the_whole_prompt(tmp_path, emulated):
    """Attention goes on from the cache by any number of tokens: a prompt in pieces of 30, 1 and
    39 tokens, a second sequence that starts while the first goes on, then single tokens; every
    position's logits equal the plain model's."""
    config = CONFIGS["B"]
    d = make_model_dir(tmp_path, config, seed=6, gain=4.0)
    w = read_weights(d)
    V = config["vocab_size"]
    a, b = random_ids(75, V, 1), random_ids(24, V, 2)
    wa, wb = plain_llama.forward_logits(config, w, a), plain_llama.forward_logits(config, w, b)
    r = build_runner(config, w, max_tokens=64 * 4, max_slots=2)
    sa, sb = r.cache.alloc_slot(), r.cache.alloc_slot()
    got = r.step([StepEntry(sa, a[:30], list(range(30)))])
    assert (got.double() - wa[:30]).abs().max() < 1e-5
    got = r.step([StepEntry(sa, a[30:31], [0])])                              # one token: a decode step
    assert (got.double() - wa[30:31]).abs().max() < 1e-5
    got = r.step([StepEntry(sa, a[31:70], list(range(39))), StepEntry(sb, b[:20], [0, 19])])
    assert (got[:39].double() - wa[31:70]).abs().max() < 1e-5
    assert (got[39:].double() - wb[[0, 19]]).abs().max() < 1e-5
    got = r.step([StepEntry(sa, a[70:], [4]), StepEntry(sb, b[20:21], [0])])   # five tokens and one
    assert (got[0].double() - wa[74]).abs().max() < 1e-5 and (got[1].double() - wb[20]).abs().max() < 1e-5
    got = r.step([StepEntry(sb, [b[21]], [0])])
    assert (got[0].double() - wb[21]).abs().max() < 1e-5
    r.cache.free_slot(sa); r.cache.free_slot(sb)
    r.cache.check()
