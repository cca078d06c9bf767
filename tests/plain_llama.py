"""Plain, slow LLaMA decoder used as the oracle of the tests.

Whole sequences, no cache, one function per part, float64 on the CPU.  Nothing
here imports the engine: the formulas are restated from the reference's text
(paths relative to the reference tree, "file:line").  Weights are a dict of
tensors under the checkpoint's own names.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


def embedding(table: torch.Tensor, ids: Sequence[int]) -> torch.Tensor:
    """Row copy without scaling: out[s, :] = table[ids[s], :].

    src/kern/naive/naive.cpp:43-54, src/core/op.cpp:55-85.
    """
    return torch.stack([table[int(i)].to(F64) for i in ids], dim=0)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """mean of squares over the row, scale by 1/sqrt(mean + eps), then the weight.

    src/kern/naive/naive.cpp:186-207 (normalise), src/core/op.cpp:37-47 (weight
    multiplied afterwards).  The reference fixes eps in code
    (src/graph/llama_like.cpp:78,96; src/core/graph.h:163); here it is an argument.
    """
    out = torch.empty_like(x, dtype=F64)
    for s in range(x.shape[0]):
        row = x[s].to(F64)
        mean = (row * row).sum() / row.numel()
        out[s] = row * (1.0 / math.sqrt(float(mean) + eps))
    return out * weight.to(F64)


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y = x . W^T with W stored [out, in], no bias.

    src/kern/naive/naive.cpp:363-379; bias=false on the LLaMA path
    (src/graph/llama_like.cpp:82, src/core/graph.cpp:63-77).
    """
    return x.to(F64) @ weight.to(F64).t()


def rope_rotate_half(u: torch.Tensor, positions: Sequence[int], theta_base: float,
                     n_rot: Optional[int] = None) -> torch.Tensor:
    """Rotate pairs (i, i + hd/2) of every head vector by the angle p * base^(-2i/n_rot).

    u: [S, heads, hd].  src/kern/naive/naive.cpp:389-414 (mode 2, "rotate half"):
    theta_i = base^(-2i/n_rot), out[i] = x0 cos - xh sin, out[i+hd/2] = x0 sin + xh cos,
    evaluated in double.  The reference fixes base = 10000 (naive.cpp:396) and
    n_rot = hd (src/graph/llama_like.cpp:60); both are arguments here.
    """
    S, H, hd = u.shape
    n_rot = hd if n_rot is None else n_rot
    half = hd // 2
    out = u.to(F64).clone()
    pos = torch.tensor([int(p) for p in positions], dtype=F64)
    for i in range(n_rot // 2):
        theta = math.pow(theta_base, (-2.0 * i) / n_rot)
        c = torch.cos(pos * theta)[:, None]
        sn = torch.sin(pos * theta)[:, None]
        x0 = u[:, :, i].to(F64)
        xh = u[:, :, i + half].to(F64)
        out[:, :, i] = x0 * c - xh * sn
        out[:, :, i + half] = x0 * sn + xh * c
    return out


def rope_interleaved(u: torch.Tensor, positions: Sequence[int], theta_base: float,
                     n_rot: Optional[int] = None) -> torch.Tensor:
    """Rotate pairs (2i, 2i+1): the other pairing the reference knows.

    src/kern/naive/naive.cpp:415-440 (mode 0): theta = base^(-i0/n_rot) for even i0.
    Not used by the LLaMA-2 graph; kept to show that the two pairings differ.
    """
    S, H, hd = u.shape
    n_rot = hd if n_rot is None else n_rot
    out = u.to(F64).clone()
    pos = torch.tensor([int(p) for p in positions], dtype=F64)
    for i0 in range(0, n_rot, 2):
        theta = math.pow(theta_base, (-1.0 * i0) / n_rot)
        c = torch.cos(pos * theta)[:, None]
        sn = torch.sin(pos * theta)[:, None]
        x0 = u[:, :, i0].to(F64)
        x1 = u[:, :, i0 + 1].to(F64)
        out[:, :, i0] = x0 * c - x1 * sn
        out[:, :, i0 + 1] = x0 * sn + x1 * c
    return out


def attention_scores(q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """s[h, a, t] = sum_d q[a, h, d] k[t, kvh(h), d], kvh(h) = h / (heads / kv_heads).

    q: [S, nh, hd], k: [L, nkv, hd].  src/kern/naive/naive.cpp:606-632 (one kv head
    per head) and :576-604 (query head h reads kv head h / heads_per_group).
    """
    S, nh, hd = q.shape
    nkv = k.shape[1]
    per_group = nh // nkv
    out = torch.empty(nh, S, k.shape[0], dtype=F64)
    for h in range(nh):
        out[h] = q[:, h, :].to(F64) @ k[:, h // per_group, :].to(F64).t()
    return out


def scale_and_causal_mask(scores: torch.Tensor, scale: float, n_past: int,
                          window: Optional[int] = None) -> torch.Tensor:
    """Multiply by the scale after the dot product; key t > n_past + a becomes -inf.

    src/kern/naive/naive.cpp:531-553, scale 1/sqrt(head size) at src/core/op.cpp:488-490.
    `window` (not in the reference) also removes keys t <= n_past + a - window.
    """
    nh, S, L = scores.shape
    out = scores * scale
    a = torch.arange(S)[:, None]
    t = torch.arange(L)[None, :]
    hidden = t > n_past + a
    if window is not None:
        hidden = hidden | (t <= n_past + a - window)
    return out.masked_fill(hidden[None, :, :], -math.inf)


def softmax_rows(scores: torch.Tensor) -> torch.Tensor:
    """Row max, exp(s - max) with -inf giving exactly 0, divide by the sum.

    src/kern/naive/naive.cpp:209-240.
    """
    m = scores.max(dim=-1, keepdim=True).values
    e = torch.where(torch.isinf(scores) & (scores < 0), torch.zeros_like(scores),
                    torch.exp(scores - m))
    return e * (1.0 / e.sum(dim=-1, keepdim=True))


def attention_context(probs: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """o[a, h, :] = sum_t p[h, a, t] v[t, kvh(h), :], heads concatenated along the row.

    src/kern/naive/naive.cpp:664-691 and :634-662 (grouped).
    """
    nh, S, L = probs.shape
    nkv, hd = v.shape[1], v.shape[2]
    per_group = nh // nkv
    out = torch.empty(S, nh, hd, dtype=F64)
    for h in range(nh):
        out[:, h, :] = probs[h] @ v[:, h // per_group, :].to(F64)
    return out.reshape(S, nh * hd)


def causal_attention(q, k, v, window: Optional[int] = None, scale: Optional[float] = None):
    """Scores, scale + mask, softmax, context for one whole sequence (n_past = 0).

    src/core/op.cpp:485-498.
    """
    hd = q.shape[-1]
    scale = 1.0 / math.sqrt(hd) if scale is None else scale
    s = attention_scores(q, k)
    s = scale_and_causal_mask(s, scale, 0, window)
    return attention_context(softmax_rows(s), v)


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)).  src/kern/naive/naive.cpp:80-89."""
    x = x.to(F64)
    return x / (1.0 + torch.exp(-x))


def swiglu_ffn(h: torch.Tensor, w_gate, w_up, w_down) -> torch.Tensor:
    """down( silu(h W1^T) * (h W3^T) ).  src/core/graph.cpp:57-79 (w1 gate, w3 up, w2 down)."""
    return linear(silu(linear(h, w_gate)) * linear(h, w_up), w_down)


def attention_block(h, positions, w, prefix, cfg, window=None):
    """q, k, v projections, rotation of q and k, attention, output projection.

    src/core/op.cpp:412-498 and src/core/graph.h:107-111.
    """
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    S = h.shape[0]
    q = linear(h, w[prefix + "self_attn.q_proj.weight"]).reshape(S, nh, hd)
    k = linear(h, w[prefix + "self_attn.k_proj.weight"]).reshape(S, nkv, hd)
    v = linear(h, w[prefix + "self_attn.v_proj.weight"]).reshape(S, nkv, hd)
    q = rope_rotate_half(q, positions, cfg["rope_theta"])
    k = rope_rotate_half(k, positions, cfg["rope_theta"])
    o = causal_attention(q, k, v, window=window)
    return linear(o, w[prefix + "self_attn.o_proj.weight"])


def decoder_layer(x, positions, w, i, cfg):
    """x1 = x + attn(norm(x)); x2 = x1 + ffn(norm(x1)).  src/graph/llama_like.cpp:66-105."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
    x1 = x + attention_block(h, positions, w, p, cfg)
    h2 = rms_norm(x1, w[p + "post_attention_layernorm.weight"], eps)
    return x1 + swiglu_ffn(h2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"])


def normalise_config(config: dict) -> dict:
    """Fill the optional keys of a LLaMA config.json (plain dict in, plain dict out)."""
    cfg = dict(config)
    cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])
    cfg.setdefault("rms_norm_eps", 1e-6)
    cfg.setdefault("rope_theta", 10000.0)
    cfg.setdefault("tie_word_embeddings", False)
    return cfg


def forward_logits(config: dict, weights: Dict[str, torch.Tensor], ids: Sequence[int]) -> torch.Tensor:
    """Logits [S, V] (float64) at every position of one whole sequence.

    Embedding, the layers, the final norm and the head (src/graph/llama_like.cpp:54-109,
    src/core/graph.cpp:117-141).  The reference's head keeps the last row only
    (src/core/op.cpp:230-274); all rows are returned here and the caller picks.
    One eps for every norm (the reference's 1e-6 / 1e-5 split is a constant of its code).
    """
    cfg = normalise_config(config)
    positions = list(range(len(ids)))
    x = embedding(weights["model.embed_tokens.weight"], ids)
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, positions, weights, i, cfg)
    x = rms_norm(x, weights["model.norm.weight"], cfg["rms_norm_eps"])
    head = weights["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] and \
        "lm_head.weight" not in weights else weights["lm_head.weight"]
    return linear(x, head)


# ---------------------------------------------------------------- sampling

def sample_top_p_top_k(logits: Sequence[float], last_n: Sequence[int], repeat_penalty: float,
                       top_k: int, top_p: float, temp: float, uniform: float) -> int:
    """The reference's sampler with the random draw given as a number in [0, 1).

    src/utils.cpp:31-115: scale by 1/temp; ids in the last-n window: negative
    logits times the penalty, others divided by it; keep the top_k largest
    (partial sort, descending); softmax in double with the max subtracted; if
    top_p < 1 keep the shortest prefix whose cumulative probability reaches top_p
    and renormalise; draw from the kept probabilities.  The draw here is the
    inverse CDF at `uniform` (the reference uses std::discrete_distribution).
    top_k <= 0 keeps every id.
    """
    scale = 1.0 / temp
    window = set(int(t) for t in last_n)
    scored = []
    for i, l in enumerate(logits):
        l = float(l)
        if i in window:
            s = l * scale * repeat_penalty if l < 0.0 else l * scale / repeat_penalty
        else:
            s = l * scale
        scored.append((s, i))
    scored.sort(key=lambda t: (-t[0], t[1]))
    if top_k > 0:
        scored = scored[:top_k]
    maxl = max(s for s, _ in scored)
    probs = [math.exp(s - maxl) for s, _ in scored]
    total = sum(probs)
    probs = [p / total for p in probs]
    if top_p < 1.0:
        cum = 0.0
        for i, p in enumerate(probs):
            cum += p
            if cum >= top_p:
                probs = probs[: i + 1]
                scored = scored[: i + 1]
                break
        probs = [p / cum for p in probs]
    cum = 0.0
    for p, (_, idx) in zip(probs, scored):
        cum += p
        if uniform < cum:
            return idx
    return scored[-1][1]


def greedy(logits: Sequence[float]) -> int:
    """Largest logit, lowest id on ties (the limit temp -> 0 of the sampler above)."""
    best, best_i = -math.inf, 0
    for i, l in enumerate(logits):
        if float(l) > best:
            best, best_i = float(l), i
    return best_i


def generate_greedy(config: dict, weights, prompt: Sequence[int], max_new_tokens: int,
                    stop_ids: Sequence[int] = ()) -> List[int]:
    """Recompute the whole sequence for every new token; stop at a stop id (not returned).

    The loop of application/chat.cpp:221-275 with the sampler replaced by argmax.
    """
    ids = list(prompt)
    out: List[int] = []
    for _ in range(max_new_tokens):
        nxt = greedy(forward_logits(config, weights, ids)[-1].tolist())
        if nxt in stop_ids:
            break
        out.append(nxt)
        ids.append(nxt)
    return out
