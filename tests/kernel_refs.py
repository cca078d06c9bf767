"""Plain torch versions of every kernel's contract (float64 inside).

Two uses: the expected side of each kernel's own test on the GPU, and, patched
over `inferllm_amd.kernels.ops` on the CPU, a stand-in that lets the step
function, the cache and the generation loop run without a GPU so that their
bookkeeping is tested where there is none.  They share no code with the kernels.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

F64 = torch.float64


def embed(tokens, table):
    return table[tokens.long()].to(torch.float32)


def add_rmsnorm(x, delta, weight, eps, out_dtype, row_idx=None):
    if delta is not None:
        if delta.dim() == 3:                           # planes of a split product
            delta = delta.to(F64).sum(0)
        s = (x.to(F64) + delta.to(F64)).to(torch.float32)
        if row_idx is None:
            x.copy_(s)
    else:
        s = x
    if row_idx is not None:
        s = s[row_idx.long()]
    v = s.to(F64)
    scale = 1.0 / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return ((v * scale) * weight.to(F64)).to(out_dtype)


def silu_mul(gate_up):
    F = gate_up.shape[1] // 2
    g, u = gate_up[:, :F].to(F64), gate_up[:, F:].to(F64)
    return (g / (1.0 + torch.exp(-g)) * u).to(gate_up.dtype)


def cache_offsets(page_table, slot, pos, page_size, ring):
    lp = pos // page_size
    if ring > 0:
        lp = lp % ring
    return int(page_table[slot, lp]), pos % page_size


def rope_store(qkv, cos_sin, rot, pairing, row_pos, row_slot, slot_len, kcache, vcache,
               page_table, page_size, ring, nh, nkv, hd):
    T = qkv.shape[0]
    view = qkv.view(T, nh + 2 * nkv, hd)
    if cos_sin is not None:
        heads = view[:, : nh + nkv, :].to(F64)
        cs = cos_sin[row_pos.long()].to(F64)          # [T, rot/2, 2]
        c, s = cs[:, None, :, 0], cs[:, None, :, 1]
        half = rot // 2
        if pairing == 0:
            a = heads[:, :, :half].clone()
            b = heads[:, :, hd // 2: hd // 2 + half].clone()
            heads[:, :, :half] = a * c - b * s
            heads[:, :, hd // 2: hd // 2 + half] = a * s + b * c
        else:
            a = heads[:, :, 0:rot:2].clone()
            b = heads[:, :, 1:rot:2].clone()
            heads[:, :, 0:rot:2] = a * c - b * s
            heads[:, :, 1:rot:2] = a * s + b * c
        view[:, : nh + nkv, :] = heads.to(qkv.dtype)
    if kcache is None:
        return
    for t in range(T):
        slot, pos = int(row_slot[t]), int(row_pos[t])
        if ring > 0 and slot_len is not None:
            last_page = (int(slot_len[slot]) - 1) // page_size
            if pos // page_size + ring <= last_page:
                continue
        page, r = cache_offsets(page_table, slot, pos, page_size, ring)
        kcache[page, :, r, :] = view[t, nh: nh + nkv, :]
        vcache[page, :, r, :] = view[t, nh + nkv:, :]


def linear(x, w, out_dtype=None):
    return (x.to(F64) @ w.to(F64).t()).to(out_dtype or x.dtype)


def qkv_rope_store_fits(x, w_qkv, hd):
    return False        # the CPU stand-in goes through linear + rope_store


def linear_add_fits(x, w, into):
    return False


def gate_up_silu(x, w_gate_up):
    return silu_mul(linear(x, w_gate_up))


def gemm_generic(x, w, out_dtype):
    return linear(x, w, out_dtype)


def _attend(q, k, v, scale, visible):
    """q [nh, hd], k/v [L, nkv, hd], visible: bool [L]."""
    nh, nkv = q.shape[0], k.shape[1]
    per = nh // nkv
    out = torch.zeros(nh, q.shape[1], dtype=F64)
    for h in range(nh):
        s = (k[:, h // per, :].to(F64) @ q[h].to(F64)) * scale
        s = s.masked_fill(~visible, -math.inf)
        p = torch.softmax(s, dim=0)
        out[h] = p @ v[:, h // per, :].to(F64)
    return out


def attn_prefill(qkv, cu_seqlens, n_seqs, max_len, nh, nkv, hd, scale, window):
    T = qkv.shape[0]
    view = qkv.view(T, nh + 2 * nkv, hd)
    out = torch.zeros(T, nh * hd, dtype=qkv.dtype, device=qkv.device)
    for b in range(n_seqs):
        s0, s1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        k, v = view[s0:s1, nh: nh + nkv], view[s0:s1, nh + nkv:]
        idx = torch.arange(s1 - s0)
        for a in range(s1 - s0):
            vis = idx <= a
            if window and window > 0:
                vis = vis & (idx > a - window)
            out[s0 + a] = _attend(view[s0 + a, :nh], k, v, scale, vis).reshape(-1).to(qkv.dtype)
    return out


def attn_prefill_paged(qkv, cu_seqlens, seq_slot, seq_start, kcache, vcache, page_table, page_size,
                       ring, n_seqs, max_len, nh, nkv, hd, scale, window):
    """Rows that go on from tokens the cache holds: row r of sequence b stands at position
    seq_start[b] + r and sees the keys 0 .. its position, all read from the paged cache."""
    T = qkv.shape[0]
    view = qkv.view(T, nh + 2 * nkv, hd)
    out = torch.zeros(T, nh * hd, dtype=qkv.dtype, device=qkv.device)
    for b in range(n_seqs):
        s0, s1 = int(cu_seqlens[b]), int(cu_seqlens[b + 1])
        if s1 == s0:
            continue
        slot, p0 = int(seq_slot[b]), int(seq_start[b])
        total = p0 + (s1 - s0)
        first = max(0, p0 - window + 1) if window and window > 0 else 0
        ks, vs = [], []
        for pos in range(first, total):
            page, r = cache_offsets(page_table, slot, pos, page_size, ring)
            ks.append(kcache[page, :, r, :])
            vs.append(vcache[page, :, r, :])
        k, v = torch.stack(ks), torch.stack(vs)
        idx = torch.arange(first, total)
        for a in range(s1 - s0):
            vis = idx <= p0 + a
            if window and window > 0:
                vis = vis & (idx > p0 + a - window)
            out[s0 + a] = _attend(view[s0 + a, :nh], k, v, scale, vis).reshape(-1).to(qkv.dtype)
    return out


def decode_splits(B, nkv, max_len, nh=0, hd=0, ragged=False):
    return 2, 1


def attn_decode(qkv, kcache, vcache, page_table, page_size, ring, seq_slot, seq_len, nh, nkv, hd,
                scale, window, nsplit, waves=1):
    B = qkv.shape[0]
    view = qkv.view(B, nh + 2 * nkv, hd)
    out = torch.zeros(B, nh * hd, dtype=qkv.dtype, device=qkv.device)
    for b in range(B):
        slot = int(seq_slot[b])
        n = int(seq_len[b])
        first = max(0, n - window) if window and window > 0 else 0
        ks, vs = [], []
        for pos in range(first, n):
            page, r = cache_offsets(page_table, slot, pos, page_size, ring)
            ks.append(kcache[page, :, r, :])
            vs.append(vcache[page, :, r, :])
        if not ks:
            continue
        k, v = torch.stack(ks), torch.stack(vs)
        vis = torch.ones(k.shape[0], dtype=torch.bool)
        out[b] = _attend(view[b, :nh], k, v, scale, vis).reshape(-1).to(qkv.dtype)
    return out


def argmax(logits):
    return torch.argmax(logits, dim=-1).to(torch.int32)   # first index on ties


def kept_distribution(logits_row, temperature, top_k, top_p, repeat_penalty, last_tokens):
    """ids kept by the sampler and their probabilities (float64), in descending order."""
    V = logits_row.numel()
    s = logits_row.to(F64) / temperature
    if last_tokens is not None:
        for t in set(int(x) for x in last_tokens if int(x) >= 0):
            s[t] = s[t] * repeat_penalty if float(logits_row[t]) < 0 else s[t] / repeat_penalty
    order = sorted(range(V), key=lambda i: (-float(s[i]), i))
    if 0 < top_k < V:
        order = order[:top_k]
    sc = torch.tensor([float(s[i]) for i in order], dtype=F64)
    p = torch.exp(sc - sc.max())
    p = p / p.sum()
    if top_p < 1.0:
        cum = torch.cumsum(p, 0)
        n = int((cum >= top_p).nonzero()[0]) + 1 if bool((cum >= top_p).any()) else len(order)
        order, p = order[:n], p[:n] / p[:n].sum()
    return order, p


_M64 = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15


def mix64(z):
    """The output function of the splitmix64 generator (public domain, Vigna): its published
    first outputs from state 0 are mix64(1 * golden), mix64(2 * golden), ... =
    0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F (pinned in the kernel tests)."""
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def uniform(seed, counter):
    """The sampler's contract, restated here and shared with nothing of the product: draw
    `counter` of a request with 64-bit `seed` uses the top 24 bits of
    mix64(seed + golden * (counter + 1)) as a number in [0, 1)."""
    return (mix64((seed + _GOLDEN * (counter + 1)) & _M64) >> 40) / 16777216.0


def sample(logits, temperature, top_k, top_p, repeat_penalty, last_tokens, seeds, counters):
    out = []
    for b in range(logits.shape[0]):
        ids, p = kept_distribution(logits[b], temperature, top_k, top_p, repeat_penalty,
                                   last_tokens[b] if last_tokens is not None else None)
        pairs = sorted(zip(ids, p.tolist()))              # inverse CDF in ascending id order
        u = uniform(int(seeds[b]) & ((1 << 64) - 1), int(counters[b]))
        cum, pick = 0.0, pairs[-1][0]
        for i, pi in pairs:
            cum += pi
            if u < cum:
                pick = i
                break
        out.append(pick)
    return torch.tensor(out, dtype=torch.int32)


def patch(monkeypatch):
    """Put these functions in place of the GPU ops (CPU tests only)."""
    from inferllm_amd.kernels import ops
    for name in ("embed", "add_rmsnorm", "silu_mul", "rope_store", "linear", "gemm_generic", "gate_up_silu", "qkv_rope_store_fits",
                 "linear_add_fits",
                 "attn_prefill", "attn_prefill_paged", "decode_splits", "attn_decode", "argmax", "sample"):
        monkeypatch.setattr(ops, name, globals()[name])
