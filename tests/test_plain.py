"""What pins the plain implementation beside the reference's text: special cases that
reduce to a library routine, invariants, and cases built so that a plausible mistake
(a wrong sign or pairing, a norm in the wrong place, a wrong eps) fails.  The reference
holds no numeric test vectors (its tests compare two back-ends on random inputs,
test/checker.cpp:46-131), so there are none to carry over: parity with the reference's
numbers is unpinned beyond these."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
from tiny import CONFIGS, TINY_A, TINY_B, make_model_dir, random_ids, read_weights

F64 = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


# ------------------------------------------------------------------ rotation
def test_rope_is_a_complex_multiplication():
    S, H, hd, base = 6, 3, 16, 10000.0
    u = rnd(S, H, hd)
    pos = [0, 1, 2, 7, 100, 4095]
    got = P.rope_rotate_half(u, pos, base)
    z = torch.complex(u[..., : hd // 2], u[..., hd // 2:])
    inv = torch.tensor([base ** (-2.0 * i / hd) for i in range(hd // 2)], dtype=F64)
    ang = torch.tensor(pos, dtype=F64)[:, None, None] * inv[None, None, :]
    w = z * torch.polar(torch.ones_like(ang), ang)               # e^{+i p theta}: a wrong sign fails
    assert torch.allclose(got[..., : hd // 2], w.real, atol=1e-12)
    assert torch.allclose(got[..., hd // 2:], w.imag, atol=1e-12)


def test_rope_invariants():
    u, v = rnd(4, 2, 24, seed=1), rnd(4, 2, 24, seed=2)
    theta = 500000.0
    assert torch.equal(P.rope_rotate_half(u, [0] * 4, theta), u)                 # position 0: identity
    r = P.rope_rotate_half(u, [3, 5, 9, 200], theta)
    assert torch.allclose(r.norm(dim=-1), u.norm(dim=-1), atol=1e-12)            # rotations keep norms
    two = P.rope_rotate_half(P.rope_rotate_half(u, [3] * 4, theta), [4] * 4, theta)
    assert torch.allclose(two, P.rope_rotate_half(u, [7] * 4, theta), atol=1e-12)  # angles add
    dots = []
    for shift in (0, 11, 1000):                                                  # only distances count
        a = P.rope_rotate_half(u, [5 + shift] * 4, theta)
        b = P.rope_rotate_half(v, [2 + shift] * 4, theta)
        dots.append((a * b).sum(-1))
    assert torch.allclose(dots[0], dots[1], atol=1e-9) and torch.allclose(dots[0], dots[2], atol=1e-9)
    assert not torch.allclose(P.rope_rotate_half(u, [1] * 4, theta), P.rope_rotate_half(u, [1] * 4, 10000.0))
    assert not torch.allclose(P.rope_rotate_half(u, [1] * 4, theta), P.rope_interleaved(u, [1] * 4, theta))


def test_interleaved_pairing_is_the_half_pairing_on_permuted_dims():
    u = rnd(3, 2, 8, seed=3)
    perm = [0, 2, 4, 6, 1, 3, 5, 7]                  # (2i, 2i+1) -> (i, i + hd/2)
    a = P.rope_interleaved(u, [1, 2, 3], 10000.0)[..., perm]
    b = P.rope_rotate_half(u[..., perm], [1, 2, 3], 10000.0)
    assert torch.allclose(a, b, atol=1e-12)


# ------------------------------------------------------------------ attention
def sdpa(q, k, v, causal):
    """torch's scaled_dot_product_attention on [heads, S, hd]."""
    return F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                          is_causal=causal).transpose(0, 1)


def test_attention_without_mask_is_the_library_routine():
    S, nh, hd = 9, 4, 16
    q, k, v = rnd(S, nh, hd, seed=1), rnd(S, nh, hd, seed=2), rnd(S, nh, hd, seed=3)
    s = P.attention_scores(q, k) * (1 / math.sqrt(hd))
    got = P.attention_context(P.softmax_rows(s), v)
    assert torch.allclose(got, sdpa(q, k, v, False).reshape(S, -1), atol=1e-10)


def test_causal_attention_one_head_and_grouped_heads():
    S, hd = 12, 24
    q, k, v = rnd(S, 1, hd, seed=4), rnd(S, 1, hd, seed=5), rnd(S, 1, hd, seed=6)
    assert torch.allclose(P.causal_attention(q, k, v), sdpa(q, k, v, True).reshape(S, -1), atol=1e-10)
    q4, k2, v2 = rnd(S, 4, hd, seed=7), rnd(S, 2, hd, seed=8), rnd(S, 2, hd, seed=9)
    rep = lambda t: t.repeat_interleave(2, dim=1)    # heads 0,1 read kv head 0; heads 2,3 kv head 1
    assert torch.allclose(P.causal_attention(q4, k2, v2),
                          sdpa(q4, rep(k2), rep(v2), True).reshape(S, -1), atol=1e-10)
    wrong = sdpa(q4, k2.repeat(1, 2, 1), v2.repeat(1, 2, 1), True).reshape(S, -1)   # h % n_kv: the other map
    assert not torch.allclose(P.causal_attention(q4, k2, v2), wrong, atol=1e-3)


def test_attention_special_cases():
    S, nh, hd = 7, 2, 8
    q, k, v = rnd(S, nh, hd, seed=1), rnd(S, nh, hd, seed=2), rnd(S, nh, hd, seed=3)
    out = P.causal_attention(q, k, v).reshape(S, nh, hd)
    assert torch.allclose(out[0], v[0], atol=1e-12)                         # one visible key: its value
    same = P.causal_attention(q, k[:1].expand(S, nh, hd), v).reshape(S, nh, hd)
    means = torch.cumsum(v, 0) / torch.arange(1, S + 1, dtype=F64)[:, None, None]
    assert torch.allclose(same, means, atol=1e-12)                          # equal keys: mean of values
    k2, v2 = k.clone(), v.clone()
    k2[5:] += 3.0; v2[5:] -= 2.0
    later = P.causal_attention(q, k2, v2).reshape(S, nh, hd)
    assert torch.equal(later[:5], out[:5]) and not torch.allclose(later[5:], out[5:])   # the future is hidden
    p = P.softmax_rows(P.scale_and_causal_mask(P.attention_scores(q, k), 0.3, 0))
    assert torch.allclose(p.sum(-1), torch.ones(nh, S, dtype=F64), atol=1e-12)
    assert float(p[:, 2, 3:].abs().max()) == 0.0                            # masked: exactly zero
    w = P.causal_attention(q, k, v, window=3).reshape(S, nh, hd)
    assert torch.allclose(w[:3], out[:3], atol=1e-12) and not torch.allclose(w[6], out[6])
    assert torch.allclose(w[6], P.causal_attention(q[4:], k[4:], v[4:]).reshape(3, nh, hd)[2], atol=1e-12)


def test_scale_is_applied_after_the_dot_product_with_head_size():
    S, nh, hd = 5, 1, 16
    q, k, v = rnd(S, nh, hd, seed=1), rnd(S, nh, hd, seed=2), rnd(S, nh, hd, seed=3)
    assert torch.allclose(P.causal_attention(q, k, v), P.causal_attention(q / 4.0, k, v, scale=1.0), atol=1e-12)


# ------------------------------------------------------------------ norm, feed-forward
def test_rms_norm_formula_and_eps():
    x, w = rnd(5, 64, seed=1) * 0.02, 1 + 0.01 * rnd(64, seed=2)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
    assert torch.allclose(P.rms_norm(x, w, 1e-6), want, atol=1e-12)
    c = torch.full((1, 8), 3.0, dtype=F64)
    assert torch.allclose(P.rms_norm(c, torch.ones(8, dtype=F64), 0.5), c / math.sqrt(9.5), atol=1e-12)
    a, b = P.rms_norm(x, w, 1e-6), P.rms_norm(x, w, 1e-5)
    assert float(((a - b).abs() / a.abs()).median()) > 5e-3          # rows of N(0, 0.02): eps shows
    assert torch.allclose(P.rms_norm(x * 7, w, 0.0), P.rms_norm(x, w, 0.0), atol=1e-9)
    centred = (x - x.mean(-1, keepdim=True))                          # a layer norm would centre: not this
    assert not torch.allclose(P.rms_norm(x, w, 1e-6), P.rms_norm(centred, w, 1e-6), atol=1e-3)


def test_swiglu_is_silu_gate_times_up():
    h, wg, wu, wd = rnd(4, 16, seed=1), rnd(40, 16, seed=2), rnd(40, 16, seed=3), rnd(16, 40, seed=4)
    want = (F.silu(h @ wg.t()) * (h @ wu.t())) @ wd.t()
    assert torch.allclose(P.swiglu_ffn(h, wg, wu, wd), want, atol=1e-10)
    swapped = (F.silu(h @ wu.t()) * (h @ wg.t())) @ wd.t()
    assert not torch.allclose(P.swiglu_ffn(h, wg, wu, wd), swapped, atol=1e-3)
    assert float(P.silu(torch.tensor([0.0]))) == 0.0 and abs(float(P.silu(torch.tensor([-40.0])))) < 1e-15
    assert abs(float(P.silu(torch.tensor([30.0]))) - 30.0) < 1e-10


def test_embedding_copies_rows():
    table = rnd(10, 128, seed=1)
    out = P.embedding(table, [1, 9, 3, 3])
    assert torch.equal(out[0], table[1]) and torch.equal(out[2], out[3]) and torch.equal(out[1], table[9])


# ------------------------------------------------------------------ whole model
@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    d = make_model_dir(tmp_path_factory.getbasetemp(), TINY_B, seed=21)
    return read_weights(d)


def test_block_is_the_identity_when_both_output_projections_are_zero(tiny):
    w = dict(tiny)
    w["model.layers.0.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.0.self_attn.o_proj.weight"])
    w["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.0.mlp.down_proj.weight"])
    x = rnd(5, 96, seed=3)
    assert torch.equal(P.decoder_layer(x, list(range(5)), w, 0, P.normalise_config(TINY_B)), x)


def test_only_distances_between_positions_count(tiny):
    cfg = P.normalise_config(TINY_B)
    x = rnd(6, 96, seed=4)
    a = P.decoder_layer(x, [0, 1, 2, 3, 4, 5], tiny, 1, cfg)
    b = P.decoder_layer(x, [100, 101, 102, 103, 104, 105], tiny, 1, cfg)
    assert torch.allclose(a, b, atol=1e-9)
    c = P.decoder_layer(x, [0, 2, 4, 6, 8, 10], tiny, 1, cfg)
    assert not torch.allclose(a, c, atol=1e-6)


def test_a_later_token_changes_no_earlier_logits_and_eps_theta_matter(tiny):
    ids = random_ids(12, 320, 1)
    base = P.forward_logits(TINY_B, tiny, ids)
    other = P.forward_logits(TINY_B, tiny, ids[:8] + [(ids[8] + 1) % 320] + ids[9:])
    assert torch.equal(other[:8], base[:8]) and not torch.allclose(other[8:], base[8:])
    assert torch.equal(P.forward_logits(TINY_B, tiny, ids[:5]), base[:5])
    for key, val in (("rms_norm_eps", 1e-6), ("rope_theta", 10000.0)):
        changed = P.forward_logits(dict(TINY_B, **{key: val}), tiny, ids)
        assert float((changed - base).abs().max() / base.abs().max()) > 1e-3


def test_head_shares_the_embedding_when_tied(tmp_path):
    cfg = CONFIGS["C"]
    w = read_weights(make_model_dir(tmp_path, cfg, seed=2))
    assert "lm_head.weight" not in w
    ids = random_ids(5, cfg["vocab_size"], 3)
    a = P.forward_logits(cfg, w, ids)
    w2 = dict(w, **{"lm_head.weight": w["model.embed_tokens.weight"].clone()})
    assert torch.equal(a, P.forward_logits(dict(cfg, tie_word_embeddings=False), w2, ids))


# ------------------------------------------------------------------ sampling
def test_sampler_follows_the_reference_steps():
    logits = [2.0, 1.0, -1.0, 0.5, 3.0, -2.0]
    assert P.greedy(logits) == 4 and P.greedy([1.0, 5.0, 5.0]) == 1
    for u in (0.0, 0.3, 0.99):
        assert P.sample_top_p_top_k(logits, [], 1.0, 1, 1.0, 0.7, u) == 4          # top_k = 1 is greedy
        assert P.sample_top_p_top_k(logits, [], 1.0, 0, 1.0, 1e-3, u) == 4         # temp -> 0 is greedy
    # descending order 4, 0, 1, 3, ...: the draw walks the cumulative probabilities
    p = torch.softmax(torch.tensor(sorted(logits, reverse=True)[:3], dtype=F64), 0).tolist()
    assert P.sample_top_p_top_k(logits, [], 1.0, 3, 1.0, 1.0, p[0] - 1e-9) == 4
    assert P.sample_top_p_top_k(logits, [], 1.0, 3, 1.0, 1.0, p[0] + 1e-9) == 0
    assert P.sample_top_p_top_k(logits, [], 1.0, 3, 1.0, 1.0, 1 - 1e-9) == 1
    # top_p keeps the shortest prefix reaching it
    full = torch.softmax(torch.tensor(sorted(logits, reverse=True), dtype=F64), 0).tolist()
    assert full[0] < 0.7 < full[0] + full[1]
    assert {P.sample_top_p_top_k(logits, [], 1.0, 0, 0.7, 1.0, u / 100) for u in range(100)} == {4, 0}
    assert {P.sample_top_p_top_k(logits, [], 1.0, 0, 0.5, 1.0, u / 100) for u in range(100)} == {4}
    # penalty: positive logits divided, negative multiplied (src/utils.cpp:46-56)
    assert P.sample_top_p_top_k([3.0, 2.9], [0], 1.3, 1, 1.0, 1.0, 0.5) == 1
    assert P.sample_top_p_top_k([-1.0, -1.2], [0], 1.3, 1, 1.0, 1.0, 0.5) == 1
    assert P.sample_top_p_top_k([-1.0, -1.2], [], 1.3, 1, 1.0, 1.0, 0.5) == 0


def test_generate_greedy_stops_at_a_stop_token(tiny):
    out = P.generate_greedy(TINY_B, tiny, [1, 5, 9], 5)
    assert len(out) == 5
    assert P.generate_greedy(TINY_B, tiny, [1, 5, 9], 5, [out[2]]) == out[:2]
