"""The cache's bookkeeping on the host: no slot or page is lost, held twice or freed
twice; groups with different needs have storage of their own; per-sequence state."""
import random

import pytest
import torch

from inferllm_amd.cache import (CacheError, CacheFull, CacheManager, FreeList, KVSpec, StateSpec)


def manager(max_tokens=64 * 8, max_slots=4, max_seq_len=256, lines=None, states=None):
    lines = lines if lines is not None else {0: KVSpec.keys_values(2, 16), 1: KVSpec.keys_values(2, 16)}
    return CacheManager(lines, states or {}, max_tokens, max_slots, max_seq_len,
                        torch.float32, "cpu")


def test_free_list_refuses_double_free_and_exhaustion():
    f = FreeList(3, "slot")
    a, b, c = f.alloc(), f.alloc(), f.alloc()
    assert sorted([a, b, c]) == [0, 1, 2]
    with pytest.raises(CacheFull):
        f.alloc()
    f.free(b)
    with pytest.raises(CacheError, match="not held"):
        f.free(b)
    with pytest.raises(CacheError, match="not held"):
        f.free(7)
    assert f.alloc() == b          # given back, used again
    f.check()


def test_slots_and_pages_are_conserved_under_random_use():
    m = manager()
    rnd = random.Random(0)
    live = {}
    for it in range(400):
        if live and rnd.random() < 0.3:
            s = rnd.choice(list(live))
            m.free_slot(s); del live[s]
        elif len(live) < 4 and rnd.random() < 0.5:
            s = m.alloc_slot(); live[s] = 0
            assert m.length(s) == 0
        elif live:
            s = rnd.choice(list(live))
            n = rnd.choice([1, 1, 1, 30, 70])
            try:
                m.extend(s, live[s], n); live[s] += n
            except CacheFull:
                pass
        m.check()
        for s, n in live.items():
            assert m.length(s) == n
            for g in m.groups:
                assert len(g.held.get(s, [])) == g.pages_needed(n)
        held = [p for g in m.groups[:1] for ps in g.held.values() for p in ps]
        assert len(held) == len(set(held))                 # no page held twice
        assert m.tokens_held() <= m.max_tokens
    for s in list(live):
        m.free_slot(s)
    assert m.slots.n_held() == 0 and all(g.pool.n_held() == 0 for g in m.groups)
    m.check()


def test_step_must_follow_the_cache():
    m = manager()
    s = m.alloc_slot()
    m.extend(s, 0, 5)
    with pytest.raises(CacheError, match="does not follow"):
        m.extend(s, 4, 1)
    with pytest.raises(CacheError, match="does not follow"):
        m.extend(s, 6, 1)
    m.extend(s, 5, 1)
    with pytest.raises(CacheFull, match="limit is 256"):
        m.extend(s, 6, 251)
    m.free_slot(s)
    with pytest.raises(CacheError, match="not held"):
        m.free_slot(s)
    with pytest.raises(CacheError, match="not held"):
        m.extend(s, 0, 1)


def test_room_is_counted_in_pages_of_64():
    m = manager(max_tokens=64 * 3, max_slots=3)
    a, b = m.alloc_slot(), m.alloc_slot()
    m.extend(a, 0, 65)        # two pages
    m.extend(b, 0, 64)        # one page
    with pytest.raises(CacheFull, match="cache full"):
        m.extend(b, 64, 1)
    m.free_slot(a)
    m.extend(b, 64, 1)        # a's pages are used again
    assert m.tokens_held() == 128
    m.check()


def test_a_step_that_does_not_fit_leaves_the_cache_as_it_was():
    m = manager(max_tokens=64 * 3, max_slots=3)
    a, b, c = m.alloc_slot(), m.alloc_slot(), m.alloc_slot()
    with pytest.raises(CacheFull, match="needs 4 more pages"):
        m.extend_all([(a, 0, 64), (b, 0, 65), (c, 0, 1)])      # a and b alone would fit
    assert [m.length(x) for x in (a, b, c)] == [0, 0, 0]
    assert all(g.pool.n_held() == 0 for g in m.groups)
    m.extend_all([(a, 0, 64), (b, 0, 64), (c, 0, 1)])
    with pytest.raises(CacheFull, match="needs 2 more pages"):
        m.extend_all([(a, 64, 1), (b, 64, 1), (c, 1, 1)])      # one of the three would fit
    assert [m.length(x) for x in (a, b, c)] == [64, 64, 1]
    with pytest.raises(CacheError, match="does not follow"):
        m.extend_all([(c, 1, 1), (a, 63, 1)])
    assert m.length(c) == 1
    m.extend_all([(c, 1, 1)])
    assert m.length(c) == 2
    m.check()


def test_groups_with_different_needs_have_their_own_storage():
    lines = {0: KVSpec.keys_values(2, 16), 1: KVSpec.keys_values(2, 16, window=70), 2: KVSpec.keys_values(4, 8),
             3: KVSpec.keys_values(2, 16, window=70)}
    m = CacheManager(lines, {}, 64 * 32, 2, 1024, torch.bfloat16, "cpu")
    assert len(m.groups) == 3
    k0, v0, g0 = m.kv_line(0)
    k1, v1, g1 = m.kv_line(1)
    k3, _, g3 = m.kv_line(3)
    assert g1 is g3 and g0 is not g1 and k1.data_ptr() != k3.data_ptr()
    assert k0.shape[1:] == (2, 64, 16) and m.kv_line(2)[0].shape[1:] == (4, 64, 8)
    assert g1.ring == 3 and g0.ring == 0                   # 70 keys touch at most 3 pages
    s = m.alloc_slot()
    m.extend(s, 0, 1000)
    assert len(g0.held[s]) == 16 and len(g1.held[s]) == 3  # the window's storage stops growing
    assert g1.n_pages == 2 * 3
    m.free_slot(s)
    m.check()


def test_page_table_and_lengths_reach_the_device_copy():
    m = manager()
    s = m.alloc_slot()
    m.extend(s, 0, 130)
    m.upload()
    g = m.groups[0]
    assert g.table[s, :3].tolist() == g.held[s] and int(g.table[s, 3]) == g.spare_page
    assert int(m.slot_len[s]) == 130
    assert g.table[m.spare_slot].tolist() == [g.spare_page] * g.pages_per_seq
    m.free_slot(s)
    m.upload()
    assert g.table[s].tolist() == [g.spare_page] * g.pages_per_seq and int(m.slot_len[s]) == 0


def test_fixed_size_state_is_zeroed_when_a_slot_is_handed_out():
    m = manager(states={1: StateSpec((3, 5), torch.float32)})
    assert m.state_line(0) is None
    st = m.state_line(1)
    assert st.shape == (5, 3, 5)
    s = m.alloc_slot()
    st[s] += 7.0
    m.free_slot(s)
    s2 = m.alloc_slot()
    assert s2 == s and float(st[s2].abs().sum()) == 0.0


def test_freed_pages_can_be_poisoned():
    m = CacheManager({0: KVSpec.keys_values(1, 8)}, {}, 128, 2, 128, torch.float32, "cpu", poison_freed=True)
    s = m.alloc_slot()
    m.extend(s, 0, 3)
    page = m.groups[0].held[s][0]
    m.free_slot(s)
    assert torch.isnan(m.kv_line(0)[0][page]).all()


def test_tokens_can_be_taken_back():
    """`rewind`: the last tokens of a sequence are given up (the void step behind a stop token);
    pages that the shorter sequence does not need go back to the pool, a window's ring keeps its
    pages, and state of fixed size refuses."""
    m = CacheManager({0: KVSpec.keys_values(2, 16), 1: KVSpec.keys_values(2, 16, window=70)}, {}, 64 * 8, 2, 512,
                     torch.float32, "cpu", poison_freed=True)
    full, ring = m.groups
    s = m.alloc_slot()
    m.extend(s, 0, 129)
    assert len(full.held[s]) == 3 and len(ring.held[s]) == 3
    third = full.held[s][2]
    m.rewind(s, 1)
    assert m.length(s) == 128 and len(full.held[s]) == 2 and len(ring.held[s]) == 2
    assert torch.isnan(m.kv_line(0)[0][third]).all() and int(full.table_host[s, 2]) == full.spare_page
    m.check()
    m.extend(s, 128, 200)                                   # the next step goes on from the shorter sequence
    assert m.length(s) == 328 and len(ring.held[s]) == 3 and len(full.held[s]) == 6
    assert ring.step_limit == 3 * 64 - 70 + 1 and m.step_limit == ring.step_limit
    with pytest.raises(CacheError, match="ring"):
        m.rewind(s, ring.step_limit + 1)                    # the ring has written over what that needs
    with pytest.raises(CacheError, match="cannot be taken back"):
        m.rewind(s, 329)
    m.rewind(s, 0)
    m.free_slot(s)
    m.check()
    with_state = CacheManager({0: KVSpec.keys_values(1, 8)}, {0: StateSpec((4,))}, 128, 2, 128, torch.float32, "cpu")
    s = with_state.alloc_slot()
    with_state.extend(s, 0, 5)
    with pytest.raises(CacheError, match="state"):
        with_state.rewind(s, 1)


def test_a_line_keeps_the_per_token_tensors_its_mixer_names():
    """Keys and values are one case: a line may keep one latent row a token, tensors of different
    widths, or a dtype of its own; lines with the same needs share a group."""
    from inferllm_amd.cache import TokenTensor
    latent = KVSpec("full", (TokenTensor("latent", (24,), torch.float32),))
    uneven = KVSpec("window", (TokenTensor("k", (2, 32)), TokenTensor("v", (2, 8), torch.float16)), window=100)
    m = CacheManager({0: latent, 1: KVSpec.keys_values(2, 16), 2: latent, 3: uneven}, {}, 64 * 8, 2, 1024,
                     torch.bfloat16, "cpu", step_rows=300)
    assert len(m.groups) == 3
    kept, g = m.token_line(2)
    assert set(kept) == {"latent"} and kept["latent"].shape == (g.n_pages + 1, 64, 24)
    assert kept["latent"].dtype == torch.float32 and g.lines == [0, 2]
    kept, g = m.token_line(3)
    assert kept["k"].shape[1:] == (2, 64, 32) and kept["k"].dtype == torch.bfloat16
    assert kept["v"].shape[1:] == (2, 64, 8) and kept["v"].dtype == torch.float16
    assert g.ring == 8 and m.step_limit == 8 * 64 - 100 + 1 >= 300   # ceil((100 - 1 + 299) / 64) + 1 pages
    k, v, _ = m.kv_line(1)
    assert k.shape[1:] == (2, 64, 16) and v.dtype == torch.bfloat16
    with pytest.raises(KeyError):
        m.kv_line(0)                                        # that line keeps no keys and values
    with pytest.raises(CacheError, match="distinct names"):
        KVSpec("full", (TokenTensor("a", (4,)), TokenTensor("a", (4,))))
    with pytest.raises(CacheError, match="positive"):
        TokenTensor("a", ())
    s = m.alloc_slot()
    m.extend(s, 0, 70)
    assert all(len(g.held[s]) == 2 for g in m.groups)
    m.free_slot(s)
    m.check()
