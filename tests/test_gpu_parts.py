"""Each part alone on the GPU against the plain functions; HIP graph replays against
eager steps; and a toy mixer with state of its own, defined here, registered, built
and stepped without a change to the framework's files."""
import math

import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def rnd(*shape, seed=0, std=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(dtype)


def make_ctx(lens_before, new_tokens, kv_lines, dtype, state_lines=None, max_slots=4, max_seq_len=512):
    """A cache and the context of one step: sequence i holds lens_before[i] tokens and gets
    new_tokens[i] more.  Returns (ctx, cache, slots)."""
    from inferllm_amd.cache import CacheManager
    from inferllm_amd.parts import StepContext
    cache = CacheManager(kv_lines, state_lines or {}, 64 * 16, max_slots, max_seq_len, dtype, DEV)
    slots = [cache.alloc_slot() for _ in lens_before]
    for s, n in zip(slots, lens_before):
        if n:
            cache.extend(s, 0, n)
    return cache, slots


def step_ctx(cache, slots, starts, counts, dtype, prefill):
    from inferllm_amd.parts import StepContext
    for s, a, n in zip(slots, starts, counts):
        cache.extend(s, a, n)
    cache.upload()
    pos = [a + j for a, n in zip(starts, counts) for j in range(n)]
    slot = [s for s, n in zip(slots, counts) for _ in range(n)]
    cu = [0]
    for n in counts:
        cu.append(cu[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return StepContext(device=DEV, act_dtype=dtype, prefill=prefill, n_rows=len(pos), n_seqs=len(slots),
                       tokens=i32([0] * len(pos)), row_pos=i32(pos), row_slot=i32(slot), cu_seqlens=i32(cu),
                       seq_slot=i32(slots), seq_len=i32([a + n for a, n in zip(starts, counts)]),
                       max_len=max(a + n for a, n in zip(starts, counts)), cache=cache)


TOL = {torch.float32: 2e-5, torch.bfloat16: 3e-2}


def rel(got, want):
    return float((got.double().cpu() - want).abs().max() / want.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,hd,E,theta,window", [(4, 2, 24, 96, 500000.0, None), (6, 6, 16, 40, 10000.0, None),
                                                        (8, 2, 64, 72, 1234.5, 21)])
def test_attention_part_whole_then_token_by_token(dtype, nh, nkv, hd, E, theta, window):
    from inferllm_amd.parts import build_part
    from inferllm_amd.config import PartSpec
    names = {"q": "q", "k": "k", "v": "v", "o": "o"}
    att = build_part("mixer", PartSpec("attention", {"hidden_size": E, "num_heads": nh, "num_kv_heads": nkv,
                                                       "head_dim": hd, "window": window, "softmax_scale": None}, names))
    rot = build_part("position", PartSpec("rotary", {"head_dim": hd, "rotary_dim": hd, "theta": theta,
                                                       "pairing": "half", "max_positions": 512}))
    w = {"q": rnd(nh * hd, E, seed=1, std=0.2), "k": rnd(nkv * hd, E, seed=2, std=0.2),
         "v": rnd(nkv * hd, E, seed=3, std=0.2), "o": rnd(E, nh * hd, seed=4, std=0.2)}
    w = {k: v.to(dtype) for k, v in w.items()}
    assert {k: tuple(v.shape) for k, v in w.items()} == {k: tuple(t.shape) for k, t in att.wants().items()}
    att.load({k: v.to(DEV) for k, v in w.items()})
    lens = [70, 5]
    hs = [rnd(n, E, seed=10 + i).to(dtype) for i, n in enumerate(lens)]

    def plain(h):
        S = h.shape[0]
        q = P.linear(h, w["q"]).reshape(S, nh, hd); k = P.linear(h, w["k"]).reshape(S, nkv, hd)
        v = P.linear(h, w["v"]).reshape(S, nkv, hd)
        q, k = P.rope_rotate_half(q, range(S), theta), P.rope_rotate_half(k, range(S), theta)
        return P.linear(P.causal_attention(q, k, v, window=window), w["o"])
    want = [plain(h) for h in hs]
    cache, slots = make_ctx([0, 0], None, {0: att.kv_spec()}, dtype)
    head = [n - 3 for n in lens]
    ctx = step_ctx(cache, slots, [0, 0], head, dtype, True)
    out = att.forward(torch.cat([h[:n] for h, n in zip(hs, head)]).to(DEV), ctx, 0, True, rot)
    assert rel(out[:head[0]], want[0][:head[0]]) < TOL[dtype] and rel(out[head[0]:], want[1][:head[1]]) < TOL[dtype]
    for j in range(3):
        ctx = step_ctx(cache, slots, [n + j for n in head], [1, 1], dtype, False)
        out = att.forward(torch.stack([h[n + j] for h, n in zip(hs, head)]).to(DEV), ctx, 0, True, rot)
        for b in range(2):
            assert rel(out[b], want[b][head[b] + j]) < TOL[dtype], (b, j)


@pytest.mark.parametrize("pairing,rot_frac", [("half", 1), ("interleaved", 1), ("half", 2)])
def test_the_decode_copy_of_qkv_follows_the_position_part(pairing, rot_frac):
    """The block tells its mixer which position encoding it has; the attention part lays the decode
    copy of q|k|v out for that encoding's fused kernel if it has one (rotate-half over the whole
    head) and in plain tiles otherwise, where the few-rows product reads it.  Either way prompt
    and single tokens equal the plain computation."""
    from inferllm_amd.config import PartSpec
    from inferllm_amd.kernels import ops
    from inferllm_amd.parts import build_part, part_class
    dtype, nh, nkv, hd, E, theta = torch.bfloat16, 4, 2, 32, 64, 10000.0
    rot_dim = hd // rot_frac
    att = build_part("mixer", PartSpec("attention", {"hidden_size": E, "num_heads": nh, "num_kv_heads": nkv,
                                                       "head_dim": hd}, {k: k for k in "qkvo"}))
    rot = build_part("position", PartSpec("rotary", {"head_dim": hd, "rotary_dim": rot_dim, "theta": theta,
                                                       "pairing": pairing, "max_positions": 512}))
    norm = lambda n: build_part("norm", PartSpec("rms_norm", {"size": E, "eps": 1e-5}, {"weight": n}))
    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": E, "intermediate_size": 128},
                                              {"gate": "g", "up": "u", "down": "d"}))
    block = part_class("block", "pre_norm")(mixer=att, feed_forward=ffn, mixer_norm=norm("n1"),
                                            feed_forward_norm=norm("n2"), position=rot)
    w = {"q": rnd(nh * hd, E, seed=1, std=0.2), "k": rnd(nkv * hd, E, seed=2, std=0.2),
         "v": rnd(nkv * hd, E, seed=3, std=0.2), "o": rnd(E, nh * hd, seed=4, std=0.2),
         "g": rnd(128, E, seed=5, std=0.2), "u": rnd(128, E, seed=6, std=0.2), "d": rnd(E, 128, seed=7, std=0.2),
         "n1": 1 + rnd(E, seed=8, std=0.1), "n2": 1 + rnd(E, seed=9, std=0.1)}
    w = {k: v.to(dtype) for k, v in w.items()}
    for part in [block] + block.parts():
        part.decode_copies = True
    block.load({k: v.to(DEV) for k, v in w.items()})
    fused = pairing == "half" and rot_frac == 1
    assert isinstance(att.w_qkv, ops.Weight) and att.w_qkv.mode == ("qkv" if fused else "plain")
    S = 9
    h = rnd(S, E, seed=20).to(dtype)

    def plain(hh):
        n = hh.shape[0]
        q = P.linear(hh, w["q"]).reshape(n, nh, hd); k = P.linear(hh, w["k"]).reshape(n, nkv, hd)
        v = P.linear(hh, w["v"]).reshape(n, nkv, hd)
        # rot_dim / 2 pairs are rotated: (i, i + head_dim / 2) or (2 i, 2 i + 1), angles by rot_dim
        rope = P.rope_rotate_half if pairing == "half" else P.rope_interleaved
        q, k = rope(q, range(n), theta, rot_dim), rope(k, range(n), theta, rot_dim)
        return P.linear(P.causal_attention(q, k, v), w["o"])
    want = plain(h)
    cache, slots = make_ctx([0], None, {0: att.kv_spec()}, dtype)
    ctx = step_ctx(cache, slots, [0], [S - 2], dtype, True)
    out = att.forward(h[:S - 2].to(DEV), ctx, 0, True, rot)
    assert rel(out, want[:S - 2]) < TOL[dtype]
    for j in (S - 2, S - 1):
        ctx = step_ctx(cache, slots, [j], [1], dtype, False)
        out = att.forward(h[j:j + 1].to(DEV), ctx, 0, True, rot)
        assert rel(out[0], want[j]) < TOL[dtype], j


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_feed_forward_and_block_parts(dtype):
    from inferllm_amd.parts import build_part, part_class
    from inferllm_amd.config import PartSpec
    E, F, eps = 72, 200, 3e-4
    norm = build_part("norm", PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": "n"}))
    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": E, "intermediate_size": F},
                                              {"gate": "g", "up": "u", "down": "d"}))
    w = {"n": (1 + rnd(E, seed=1, std=0.1)).to(dtype), "g": rnd(F, E, seed=2, std=0.2).to(dtype),
         "u": rnd(F, E, seed=3, std=0.2).to(dtype), "d": rnd(E, F, seed=4, std=0.2).to(dtype)}
    for p in (norm, ffn):
        p.load({k: v.to(DEV) for k, v in w.items()})
    cache, slots = make_ctx([0], None, {}, dtype)
    ctx = step_ctx(cache, slots, [0], [9], dtype, True)
    x, delta = rnd(9, E, seed=5, std=0.05), rnd(9, E, seed=6, std=0.05).to(dtype)
    xg = x.to(DEV)
    h = norm.forward(xg, delta.to(DEV), ctx)
    want_x = x.double() + delta.double()
    assert rel(xg, want_x) < 1e-6 and h.dtype == dtype                      # the residual stays float32
    assert rel(h, P.rms_norm(want_x, w["n"], eps)) < TOL[dtype]
    out = ffn.forward(h, ctx)
    assert rel(out, P.swiglu_ffn(h.cpu(), w["g"], w["u"], w["d"])) < TOL[dtype]


def test_feed_forward_adds_to_the_stream_and_prepares_the_next_norm():
    """The short cut of few bfloat16 rows: the feed-forward adds its output to the residual rows
    itself and hands on rows prepared for the norm that follows; a block takes them only for
    the norm they were made for, and a part that does not take them gets plain normed rows."""
    from inferllm_amd.parts import build_part
    from inferllm_amd.parts.block import PreNormBlock
    from inferllm_amd.config import PartSpec
    from inferllm_amd.kernels import ops
    dtype, E, F, eps = torch.bfloat16, 64, 96, 1e-5
    mk_norm = lambda name: build_part("norm", PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": name}))
    n_next, n_other = mk_norm("n1"), mk_norm("n2")
    ffn = build_part("feed_forward", PartSpec("swiglu", {"hidden_size": E, "intermediate_size": F},
                                              {"gate": "g", "up": "u", "down": "d"}))
    w = {"n1": (1 + rnd(E, seed=1, std=0.2)).to(dtype), "n2": (1 + rnd(E, seed=7, std=0.2)).to(dtype),
         "g": rnd(F, E, seed=2, std=0.2).to(dtype), "u": rnd(F, E, seed=3, std=0.2).to(dtype),
         "d": rnd(E, F, seed=4, std=0.2).to(dtype)}
    for p in (n_next, n_other, ffn):
        p.load({k: v.to(DEV) for k, v in w.items()})
    cache, slots = make_ctx([0], None, {}, dtype)
    ctx = step_ctx(cache, slots, [0], [5], dtype, False)
    x = rnd(5, E, seed=5, std=0.5)
    h = rnd(5, E, seed=6, std=0.5).to(dtype)
    want_x = x.double() + P.swiglu_ffn(h, w["g"], w["u"], w["d"])
    xg = x.to(DEV)
    rows = ffn.forward(h.to(DEV), ctx, residual=xg, next_norm=n_next)
    assert isinstance(rows, ops.NormedRows) and rows.x is xg
    assert rel(xg, want_x) < TOL[dtype]                                   # the sum is in the stream
    takes = type("Takes", (), {"takes_normed_rows": True})()
    plain = type("Plain", (), {"takes_normed_rows": False})()
    assert PreNormBlock._enter(n_next, takes, xg, rows, ctx) is rows       # made for this norm
    got = PreNormBlock._enter(n_next, plain, xg, rows, ctx)                # a part that wants rows
    assert rel(got, P.rms_norm(want_x, w["n1"], eps)) < TOL[dtype]
    got = PreNormBlock._enter(n_other, takes, xg, rows, ctx)               # made for another norm
    assert isinstance(got, torch.Tensor) and rel(got, P.rms_norm(want_x, w["n2"], eps)) < TOL[dtype]
    assert rel(xg, want_x) < TOL[dtype]                                   # and nothing was added twice
    # the product of the prepared rows is the product of the normed rows
    wq = rnd(40, E, seed=9, std=0.2).to(dtype)
    want = P.linear(P.rms_norm(want_x, w["n1"], eps), wq)
    assert rel(ops.linear(rows, wq.to(DEV)), want) < TOL[dtype]


@pytest.mark.parametrize("n_reqs", [3, 20])
def test_decode_graph_replays_equal_eager_steps(tmp_path, n_reqs):
    """The same decode steps through the captured HIP graph (replayed many times, with other
    work and synchronisations between) and eagerly: every replay equals its eager step."""
    import inferllm_amd as I
    from tiny import TINY_B, make_model_dir, random_ids
    d = make_model_dir(tmp_path, TINY_B, seed=3, dtype=torch.bfloat16)
    reqs = [random_ids(n, 320, n) for n in ([30, 12, 50] + list(range(13, 30)))[:n_reqs]]
    outs = []
    for graphs in (True, False):
        eng = I.Engine.from_pretrained(d, dtype="bfloat16", max_batch=n_reqs, use_graphs=graphs)
        slots = [eng.alloc_slot() for _ in reqs]
        eng.step([I.StepEntry(s, r[:10], []) for s, r in zip(slots, reqs)])
        seq = []
        for j in range(10, 30):
            live = [(s, r) for s, r in zip(slots, reqs) if j < len(r)]
            seq.append(eng.step([I.StepEntry(s, [r[j]], [0]) for s, r in live]).clone())
            torch.cuda.synchronize()
            junk = torch.randn(256, 256, device="cuda:0") @ torch.randn(256, 256, device="cuda:0")
            junk.sum().item()
        outs.append(seq)
    for a, b in zip(*outs):
        assert a.shape == b.shape and torch.equal(a, b)


# ---------------------------------------------------------------- a toy mixer with state
_toy = []


def register_toy():
    """Registers the toy parts and architecture once a process; returns the config class."""
    if not _toy:
        _toy.append(_register_toy())
    return _toy[0]


def _register_toy():
    from inferllm_amd.cache import StateSpec
    from inferllm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferllm_amd.parts import Mixer, register_part
    from inferllm_amd.weights import TensorWant

    @register_part("mixer", "toy_running_mean")
    class RunningMean(Mixer):
        """delta_t = W . mean(h_0 .. h_t): the sum and the count live in per-sequence state."""
        graph_safe = False          # reads lengths on the host

        def __init__(self, hidden_size, tensors=None):
            super().__init__(tensors)
            self.E = hidden_size

        def shapes(self):
            return {"w": TensorWant((self.E, self.E))}

        def state_spec(self):
            return StateSpec((self.E + 1,), torch.float32)

        def load(self, tensors):
            self.w = self._take(tensors, "w").float()

        def forward(self, h, ctx, line, writes_cache, position):
            state = ctx.cache.state_line(line)
            cu, slots = ctx.cu_seqlens.tolist(), ctx.seq_slot.tolist()
            out = torch.empty(h.shape, dtype=torch.float32, device=h.device)
            for b, s in enumerate(slots):
                rows = h[cu[b]:cu[b + 1]].float()
                sums = state[s, :self.E] + torch.cumsum(rows, 0)
                counts = state[s, self.E] + torch.arange(1, rows.shape[0] + 1, device=h.device)
                out[cu[b]:cu[b + 1]] = sums / counts[:, None]
                state[s, :self.E] = sums[-1]
                state[s, self.E] = counts[-1]
            return (out @ self.w.t()).to(h.dtype)

    @register_part("mixer", "toy_running_mean_on_device")
    class RunningMeanOnDevice(RunningMean):
        """The same with steps of single tokens done on the device alone (no host read), so that
        they may be captured into a graph; and it goes on from its state by any number of tokens."""
        graph_safe = True
        takes_continuations = True

        def forward(self, h, ctx, line, writes_cache, position):
            if ctx.prefill:
                return super().forward(h, ctx, line, writes_cache, position)
            state = ctx.cache.state_line(line)
            slots = ctx.seq_slot.long()
            now = state.index_select(0, slots)
            now[:, :self.E] += h.float()
            now[:, self.E] += 1
            state.index_copy_(0, slots, now)
            return ((now[:, :self.E] / now[:, self.E:]) @ self.w.t()).to(h.dtype)

    @register_architecture("ToyRunningMeanForTests")
    class ToyConfig:
        def __init__(self, hidden_size, vocab_size, layers, eps, mixer="toy_running_mean"):
            self.E, self.V, self.L, self.eps, self.mixer = hidden_size, vocab_size, layers, eps, mixer

        @classmethod
        def from_dict(cls, d):
            return cls(d["hidden_size"], d["vocab_size"], d["layers"], d["eps"],
                       d.get("mixer", "toy_running_mean"))

        def to_dict(self):
            return {"architectures": ["ToyRunningMeanForTests"], "hidden_size": self.E,
                    "vocab_size": self.V, "layers": self.L, "eps": self.eps, "mixer": self.mixer}

        def to_spec(self):
            norm = lambda n: PartSpec("rms_norm", {"size": self.E, "eps": self.eps}, {"weight": n})
            layers = [LayerSpec("pre_norm", PartSpec(self.mixer, {"hidden_size": self.E}, {"w": f"l{i}.mix"}),
                                PartSpec("swiglu", {"hidden_size": self.E, "intermediate_size": 2 * self.E},
                                         {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                                norm(f"l{i}.n1"), norm(f"l{i}.n2"), None) for i in range(self.L)]
            return ModelSpec("ToyRunningMeanForTests", self.V, self.E, 4096,
                             PartSpec("token_embedding", {"vocab_size": self.V, "hidden_size": self.E}, {"weight": "emb"}),
                             layers, [ScheduleEntry(i, i) for i in range(self.L)], norm("nf"),
                             PartSpec("lm_head", {"hidden_size": self.E, "vocab_size": self.V}, {"weight": "head"}))
    return ToyConfig


def toy_plain(w, cfg, ids):
    x = P.embedding(w["emb"], ids)
    for i in range(cfg["layers"]):
        h = P.rms_norm(x, w[f"l{i}.n1"], cfg["eps"])
        mean = torch.cumsum(h, 0) / torch.arange(1, len(ids) + 1, dtype=torch.float64)[:, None]
        x = x + P.linear(mean, w[f"l{i}.mix"])
        x = x + P.swiglu_ffn(P.rms_norm(x, w[f"l{i}.n2"], cfg["eps"]), w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])
    return P.linear(P.rms_norm(x, w["nf"], cfg["eps"]), w["head"])


def test_a_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    import inferllm_amd as I
    from tiny import random_ids, read_weights
    register_toy()
    cfg = {"architectures": ["ToyRunningMeanForTests"], "hidden_size": 48, "vocab_size": 100, "layers": 2, "eps": 1e-5}
    d = I.write_random_model(str(tmp_path / "toy"), I.config_from_dict(cfg), seed=4)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="float32", max_batch=2, max_seq_len=256)
    assert not eng.cache.groups and set(eng.cache.states) == {0, 1}          # state, and no keys at all
    reqs = [random_ids(n, 100, n) for n in (20, 7, 33)]
    want = [toy_plain(w, cfg, r) for r in reqs]
    for order in ([0, 1], [2, 1]):                                           # slots are used again: state starts at zero
        slots = {i: eng.alloc_slot() for i in order}
        head = {i: len(reqs[i]) - 4 for i in order}
        out = eng.step([I.StepEntry(slots[i], reqs[i][:head[i]], [head[i] - 1]) for i in order])
        for j, i in enumerate(order):
            assert rel(out[j], want[i][head[i] - 1]) < 2e-5
        for t in range(4):
            out = eng.step([I.StepEntry(slots[i], [reqs[i][head[i] + t]], [0]) for i in order])
            for j, i in enumerate(order):
                assert rel(out[j], want[i][head[i] + t]) < 2e-5
        for i in order:
            eng.free_slot(slots[i])
    got = eng.generate([reqs[1]], max_new_tokens=3, stop_token_ids=[])
    seq = list(reqs[1])
    for _ in range(3):
        seq.append(int(torch.argmax(toy_plain(w, cfg, seq)[-1])))
    assert got == [seq[len(reqs[1]):]]


@pytest.mark.parametrize("graphs", [True, False])
def test_a_mixer_with_state_under_decode_graphs(tmp_path, graphs):
    """State is not idempotent as a store of keys is: a decode step that ran twice (once to warm
    up before the capture of its graph, once as the replay) would count a token twice.  Steps of
    1, 2 and 3 sequences (three graphs, each captured at its first use, in the middle of the
    sequences) must leave the running means as one pass over the tokens does."""
    import inferllm_amd as I
    from tiny import random_ids, read_weights
    register_toy()
    cfg = {"architectures": ["ToyRunningMeanForTests"], "hidden_size": 48, "vocab_size": 100, "layers": 2,
           "eps": 1e-5, "mixer": "toy_running_mean_on_device"}
    d = I.write_random_model(str(tmp_path / "toy"), I.config_from_dict(cfg), seed=4)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="float32", max_batch=4, max_seq_len=256, use_graphs=graphs)
    assert eng.runner.use_graphs == graphs
    reqs = [random_ids(n, 100, 40 + n) for n in (12, 9, 15)]
    want = [toy_plain(w, cfg, r) for r in reqs]
    slots = [eng.alloc_slot() for _ in reqs]
    heads = [3, 2, 4]
    eng.step([I.StepEntry(s, r[:h], []) for s, r, h in zip(slots, reqs, heads)])
    at = list(heads)
    live = [0, 1, 2]
    while live:
        out = eng.step([I.StepEntry(slots[i], [reqs[i][at[i]]], [0]) for i in live])
        for j, i in enumerate(live):
            assert rel(out[j], want[i][at[i]]) < 2e-5, (i, at[i], len(live))
            at[i] += 1
        live = [i for i in live if at[i] < len(reqs[i])]
    if graphs:
        assert {k[0] for k in eng.runner._graphs} == {1, 2, 4}


def test_prompt_steps_are_replayed_from_graphs_only_if_every_part_says_so(tmp_path):
    """A part that promises no host reads in steps of single tokens (`graph_safe`) has promised
    nothing about steps of several tokens: the toy mixer reads the step's lengths on the host
    there, which a capture would refuse.  Its model's short prompt steps run eagerly however
    often a shape comes back, while its decode steps are replayed from graphs; a model of the
    library's own parts has both."""
    import inferllm_amd as I
    from tiny import TINY_A, make_model_dir, random_ids, read_weights
    register_toy()
    cfg = {"architectures": ["ToyRunningMeanForTests"], "hidden_size": 48, "vocab_size": 100, "layers": 2,
           "eps": 1e-5, "mixer": "toy_running_mean_on_device"}
    d = I.write_random_model(str(tmp_path / "toy"), I.config_from_dict(cfg), seed=8)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="float32", max_batch=2, max_seq_len=256)
    assert eng.runner.use_graphs and not eng.runner.use_prompt_graphs
    for turn in range(3):                                   # the same shapes three times
        ids = random_ids(14, 100, 60 + turn)
        want = toy_plain(w, cfg, ids)
        s = eng.alloc_slot()
        out = eng.step([I.StepEntry(s, ids[:9], [0, 8])])
        assert rel(out[0], want[0]) < 2e-5 and rel(out[1], want[8]) < 2e-5
        out = eng.step([I.StepEntry(s, ids[9:12], [2])])    # goes on by three tokens
        assert rel(out[0], want[11]) < 2e-5
        for t in (12, 13):
            assert rel(eng.step([I.StepEntry(s, [ids[t]], [0])])[0], want[t]) < 2e-5
        eng.free_slot(s)
    assert not eng.runner._prompt_graphs and {k[0] for k in eng.runner._graphs} == {1}
    la = I.Engine.from_pretrained(make_model_dir(tmp_path, TINY_A, seed=1), dtype="float32", max_batch=2)
    assert la.runner.use_prompt_graphs


def test_a_mixer_says_whether_it_goes_on_by_several_tokens(tmp_path):
    """The rule "all start, or all go on by one" belongs to the mixers: a mixer that says it takes
    continuations (one with state of fixed size here; attention without a window too) lets a
    prompt be cut into steps of any lengths, also mixed with sequences that start; a model with
    a mixer that does not is refused such steps."""
    import inferllm_amd as I
    from inferllm_amd.engine.step import StepError
    from tiny import TINY_A, make_model_dir, random_ids, read_weights
    register_toy()
    cfg = {"architectures": ["ToyRunningMeanForTests"], "hidden_size": 48, "vocab_size": 100, "layers": 2,
           "eps": 1e-5, "mixer": "toy_running_mean_on_device"}
    d = I.write_random_model(str(tmp_path / "toy"), I.config_from_dict(cfg), seed=6)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="float32", max_batch=4, max_seq_len=256)
    a, b = random_ids(30, 100, 1), random_ids(11, 100, 2)
    wa, wb = toy_plain(w, cfg, a), toy_plain(w, cfg, b)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    out = eng.step([I.StepEntry(sa, a[:7], [6])])
    assert rel(out[0], wa[6]) < 2e-5
    out = eng.step([I.StepEntry(sa, a[7:20], [0, 12]), I.StepEntry(sb, b[:5], [4])])   # one goes on, one starts
    assert rel(out[0], wa[7]) < 2e-5 and rel(out[1], wa[19]) < 2e-5 and rel(out[2], wb[4]) < 2e-5
    out = eng.step([I.StepEntry(sa, a[20:], [9]), I.StepEntry(sb, b[5:6], [0])])       # ten tokens and one
    assert rel(out[0], wa[29]) < 2e-5 and rel(out[1], wb[5]) < 2e-5
    # the host-reading form of the mixer does not say it can: the step function refuses and says
    # which part is the reason; attention without a window can (tests/test_gpu_model.py)
    cfg2 = dict(cfg, mixer="toy_running_mean")
    d2 = I.write_random_model(str(tmp_path / "toy2"), I.config_from_dict(cfg2), seed=6)
    e2 = I.Engine.from_pretrained(d2, dtype="float32", max_batch=2, max_seq_len=256)
    s = e2.alloc_slot()
    e2.step([I.StepEntry(s, [1, 2, 3], [])])
    with pytest.raises(StepError, match="RunningMean cannot go on by several"):
        e2.step([I.StepEntry(s, [4, 5], [1])])
    assert e2.cache.length(s) == 3                       # refused before anything was reserved
    la = I.Engine.from_pretrained(make_model_dir(tmp_path, TINY_A, seed=1), dtype="float32", max_batch=2)
    assert la.model.one_token_mixers == []


def test_embedding_and_head_parts():
    from inferllm_amd.parts import build_part
    from inferllm_amd.config import PartSpec
    V, E = 411, 80
    emb = build_part("embedding", PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E}, {"weight": "e"}))
    head = build_part("head", PartSpec("lm_head", {"hidden_size": E, "vocab_size": V, "tied_fallback": "e"}, {"weight": "h"}))
    w = rnd(V, E, seed=1, std=0.3).to(torch.bfloat16)
    assert head.wants()["h"].optional and not head.wants()["e"].optional
    emb.load({"e": w.to(DEV)}); head.load({"e": w.to(DEV)})
    cache, slots = make_ctx([0], None, {}, torch.bfloat16)
    ctx = step_ctx(cache, slots, [0], [4], torch.bfloat16, True)
    ctx.tokens = torch.tensor([5, 0, 410, 5], dtype=torch.int32, device=DEV)
    x = emb.forward(ctx)
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), w[[5, 0, 410, 5]].float())
    h = rnd(4, E, seed=2).to(torch.bfloat16)
    logits = head.forward(h.to(DEV), ctx)
    assert logits.dtype == torch.float32 and rel(logits, P.linear(h, w)) < 1e-4     # float32 out of bfloat16 operands


def test_schedule_runs_a_layer_twice_and_shares_a_cache_line(tmp_path):
    """The order of layers is data: layer 0 runs twice (two cache lines), then layer 1 reads the
    keys and values that layer 0's second run stored.  Whole, token by token and in a batch."""
    import inferllm_amd as I
    from inferllm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from tiny import random_ids, read_weights
    E, V, nh, nkv, hd, F, eps, theta = 64, 90, 4, 2, 16, 100, 1e-5, 10000.0

    @register_architecture("ToyScheduleForTests")
    class Cfg:
        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyScheduleForTests"]}

        def to_spec(self):
            norm = lambda n: PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": n})
            def layer(i):
                return LayerSpec("pre_norm",
                                 PartSpec("attention", {"hidden_size": E, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd},
                                          {k: f"l{i}.{k}" for k in "qkvo"}),
                                 PartSpec("swiglu", {"hidden_size": E, "intermediate_size": F},
                                          {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                                 norm(f"l{i}.n1"), norm(f"l{i}.n2"),
                                 PartSpec("rotary", {"head_dim": hd, "rotary_dim": hd, "theta": theta, "pairing": "half",
                                                     "max_positions": 256}))
            sched = [ScheduleEntry(0, 0), ScheduleEntry(0, 1), ScheduleEntry(1, 1, writes_cache=False)]
            return ModelSpec("ToyScheduleForTests", V, E, 256,
                             PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E}, {"weight": "emb"}),
                             [layer(0), layer(1)], sched, norm("nf"),
                             PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "head"}))

    d = I.write_random_model(str(tmp_path / "sched"), Cfg(), seed=8)
    w = read_weights(d)

    def plain(ids):
        S = len(ids)
        pos = list(range(S))
        def attn(i, h, kv=None):
            q = P.rope_rotate_half(P.linear(h, w[f"l{i}.q"]).reshape(S, nh, hd), pos, theta)
            if kv is None:
                k = P.rope_rotate_half(P.linear(h, w[f"l{i}.k"]).reshape(S, nkv, hd), pos, theta)
                v = P.linear(h, w[f"l{i}.v"]).reshape(S, nkv, hd)
            else:
                k, v = kv
            return P.linear(P.causal_attention(q, k, v), w[f"l{i}.o"]), (k, v)
        def block(i, x, kv=None):
            d1, kv = attn(i, P.rms_norm(x, w[f"l{i}.n1"], eps), kv)
            x = x + d1
            return x + P.swiglu_ffn(P.rms_norm(x, w[f"l{i}.n2"], eps), w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"]), kv
        x = P.embedding(w["emb"], ids)
        x, _ = block(0, x)
        x, kv = block(0, x)
        x, _ = block(1, x, kv)
        return P.linear(P.rms_norm(x, w["nf"], eps), w["head"])

    eng = I.Engine.from_pretrained(d, dtype="float32", max_batch=2, max_seq_len=128)
    assert len(eng.cache.groups) == 1 and eng.cache.groups[0].lines == [0, 1]
    reqs = [random_ids(n, V, n) for n in (30, 9)]
    want = [plain(r) for r in reqs]
    slots = [eng.alloc_slot(), eng.alloc_slot()]
    head = [len(r) - 3 for r in reqs]
    out = eng.step([I.StepEntry(s, r[:n], list(range(n))) for s, r, n in zip(slots, reqs, head)])
    assert rel(out[:head[0]], want[0][:head[0]]) < 2e-5 and rel(out[head[0]:], want[1][:head[1]]) < 2e-5
    for j in range(3):
        out = eng.step([I.StepEntry(s, [r[n + j]], [0]) for s, r, n in zip(slots, reqs, head)])
        for b in range(2):
            assert rel(out[b], want[b][head[b] + j]) < 2e-5, (b, j)


def test_toy_routed_feed_forward_and_learned_positions(tmp_path):
    """Two more toy parts defined here: a feed-forward that routes every row to one of three
    experts (router logits in float32, top-1), and a position encoding that adds a learned table
    to the embedded rows and leaves q and k alone.  Registered, built from a spec, stepped whole,
    token by token and in a batch, against a plain computation."""
    import inferllm_amd as I
    from inferllm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferllm_amd.kernels import ops
    from inferllm_amd.parts import FeedForward, PositionEncoding, register_part
    from inferllm_amd.weights import TensorWant
    from tiny import random_ids, read_weights
    E, V, nh, hd, F, X, eps, P_MAX = 48, 70, 3, 16, 64, 3, 1e-5, 128

    @register_part("feed_forward", "toy_top1_experts")
    class Top1Experts(FeedForward):
        graph_safe = False              # routes on the host

        def __init__(self, hidden_size, intermediate_size, experts, tensors=None):
            super().__init__(tensors)
            self.E, self.F, self.X = hidden_size, intermediate_size, experts

        def shapes(self):
            out = {"router": TensorWant((self.X, self.E))}
            for x in range(self.X):
                out[f"gate_up{x}"] = TensorWant((2 * self.F, self.E))
                out[f"down{x}"] = TensorWant((self.E, self.F))
            return out

        def load(self, tensors):
            self.router = self._take(tensors, "router")
            self.gu = [self._take(tensors, f"gate_up{x}") for x in range(self.X)]
            self.down = [self._take(tensors, f"down{x}") for x in range(self.X)]

        def forward(self, h, ctx):
            logits = ops.linear(h, self.router, out_dtype=torch.float32)     # router in float32
            choice = torch.argmax(logits, dim=-1)
            out = torch.zeros_like(h)
            for x in range(self.X):
                rows = (choice == x).nonzero().flatten()
                if rows.numel():
                    hx = h[rows].contiguous()
                    out[rows] = ops.linear(ops.gate_up_silu(hx, self.gu[x]), self.down[x])
            return out

    @register_part("position", "toy_learned_absolute")
    class LearnedAbsolute(PositionEncoding):
        def __init__(self, hidden_size, max_positions, tensors=None):
            super().__init__(tensors)
            self.E, self.P = hidden_size, max_positions

        def shapes(self):
            return {"table": TensorWant((self.P, self.E))}

        def load(self, tensors):
            self.table = self._take(tensors, "table").float()

        def on_embedding(self, x, ctx):
            x += self.table[ctx.row_pos.long()]

        def on_qkv(self, qkv, ctx, nh, nkv, hd, kcache, vcache, group):
            ops.rope_store(qkv, None, 0, 0, ctx.row_pos, ctx.row_slot,
                           ctx.cache.slot_len if ctx.prefill else None, kcache, vcache,
                           group.table if group is not None else None,
                           group.page_size if group is not None else 1,
                           group.ring if group is not None else 0, nh, nkv, hd)

    @register_architecture("ToyRoutedForTests")
    class Cfg:
        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyRoutedForTests"]}

        def to_spec(self):
            norm = lambda n: PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": n})
            pos = PartSpec("toy_learned_absolute", {"hidden_size": E, "max_positions": P_MAX}, {"table": "pos"})
            def ffn(i):
                t = {"router": f"l{i}.router"}
                for x in range(X):
                    t[f"gate_up{x}"] = f"l{i}.x{x}.gu"; t[f"down{x}"] = f"l{i}.x{x}.d"
                return PartSpec("toy_top1_experts", {"hidden_size": E, "intermediate_size": F, "experts": X}, t)
            layers = [LayerSpec("pre_norm",
                                PartSpec("attention", {"hidden_size": E, "num_heads": nh, "num_kv_heads": nh, "head_dim": hd},
                                         {k: f"l{i}.{k}" for k in "qkvo"}),
                                ffn(i) if i == 1 else PartSpec("swiglu", {"hidden_size": E, "intermediate_size": F},
                                                                {"gate": "l0.g", "up": "l0.u", "down": "l0.d"}),
                                norm(f"l{i}.n1"), norm(f"l{i}.n2"), pos) for i in range(2)]
            return ModelSpec("ToyRoutedForTests", V, E, P_MAX,
                             PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E}, {"weight": "emb"}),
                             layers, [ScheduleEntry(0, 0), ScheduleEntry(1, 1)], norm("nf"),
                             PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "head"}))

    d = I.write_random_model(str(tmp_path / "routed"), Cfg(), seed=6)
    w = read_weights(d)
    w["pos"] = w["pos"] * 20.0                                  # positions must matter
    w["l1.router"] = w["l1.router"] * 50.0                      # clear choices, all experts used
    from inferllm_amd.weights import write_safetensors
    write_safetensors(str(tmp_path / "routed" / "model.safetensors"), w.items())

    def plain(ids):
        S = len(ids)
        x = P.embedding(w["emb"], ids) + w["pos"][:S].double()
        used = set()
        for i in range(2):
            h = P.rms_norm(x, w[f"l{i}.n1"], eps)
            q, k, v = (P.linear(h, w[f"l{i}.{n}"]).reshape(S, nh, hd) for n in "qkv")
            x = x + P.linear(P.causal_attention(q, k, v), w[f"l{i}.o"])
            h = P.rms_norm(x, w[f"l{i}.n2"], eps)
            if i == 0:
                x = x + P.swiglu_ffn(h, w["l0.g"], w["l0.u"], w["l0.d"])
            else:
                choice = torch.argmax(P.linear(h, w["l1.router"]), dim=-1)
                y = torch.zeros_like(x)
                for r in range(S):
                    e = int(choice[r]); used.add(e)
                    gu = w[f"l1.x{e}.gu"]
                    y[r] = P.swiglu_ffn(h[r:r + 1], gu[:F], gu[F:], w[f"l1.x{e}.d"])[0]
                x = x + y
        return P.linear(P.rms_norm(x, w["nf"], eps), w["head"]), used

    eng = I.Engine.from_pretrained(d, dtype="float32", max_batch=2, max_seq_len=P_MAX)
    assert not eng.runner.use_graphs                            # a part of the model reads on the host
    reqs = [random_ids(n, V, 3 * n) for n in (40, 11)]
    want = [plain(r) for r in reqs]
    assert want[0][1] == {0, 1, 2}                              # every expert had rows
    slots = [eng.alloc_slot(), eng.alloc_slot()]
    head = [len(r) - 3 for r in reqs]
    out = eng.step([I.StepEntry(s, r[:n], list(range(n))) for s, r, n in zip(slots, reqs, head)])
    assert rel(out[:head[0]], want[0][0][:head[0]]) < 2e-5 and rel(out[head[0]:], want[1][0][:head[1]]) < 2e-5
    for j in range(3):
        out = eng.step([I.StepEntry(s, [r[n + j]], [0]) for s, r, n in zip(slots, reqs, head)])
        for b in range(2):
            assert rel(out[b], want[b][0][head[b] + j]) < 2e-5, (b, j)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_and_toy_arrangement_of_a_block(tmp_path, dtype):
    """The last two kinds of parts as toys of the test: a norm that subtracts the mean and has a
    bias (float32 statistics, no planes, nothing a product's kernel may take over), and a block
    in which mixer and feed-forward read the same normed rows and both results are added.
    Registered, built from a spec next to a layer of the library's own parts, stepped whole and
    token by token in a batch of two, under decode graphs, against a plain computation."""
    import inferllm_amd as I
    from inferllm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferllm_amd.parts import Block, Norm, register_part
    from inferllm_amd.weights import TensorWant, write_safetensors
    from tiny import random_ids, read_weights
    E, V, nh, nkv, hd, F, eps, P_MAX, theta = 64, 90, 4, 2, 16, 96, 1e-4, 96, 5000.0

    @register_part("norm", "toy_layer_norm_" + dtype)
    class ToyLayerNorm(Norm):
        def __init__(self, size, eps, tensors=None):
            super().__init__(tensors)
            self.size, self.eps = size, eps

        def shapes(self):
            return {"weight": TensorWant((self.size,), init="ones_normal", keep_stored=True),
                    "bias": TensorWant((self.size,), keep_stored=True)}

        def load(self, tensors):
            self.weight = self._take(tensors, "weight").float()
            self.bias = self._take(tensors, "bias").float()

        def forward(self, x, delta, ctx, row_idx=None):
            if row_idx is None:
                if delta is not None:
                    x.add_(delta.float())
                rows = x
            else:
                rows = x[row_idx.long()]
                if delta is not None:
                    rows = rows + delta[row_idx.long()].float()
            mean = rows.mean(dim=-1, keepdim=True)
            var = ((rows - mean) ** 2).mean(dim=-1, keepdim=True)
            return ((rows - mean) * torch.rsqrt(var + self.eps) * self.weight + self.bias).to(ctx.act_dtype)

    @register_part("block", "toy_parallel_" + dtype)
    class ToyParallelBlock(Block):
        def forward(self, x, pending, ctx, line, writes_cache):
            h = self.mixer_norm.forward(x, pending, ctx)
            a = self.mixer.forward(h, ctx, line, writes_cache, self.position)
            return a.float() + self.feed_forward.forward(h, ctx).float()

    @register_architecture("ToyParallelForTests_" + dtype)
    class Cfg:
        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyParallelForTests_" + dtype]}

        def to_spec(self):
            rms = lambda n: PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": n})
            ln = lambda n: PartSpec("toy_layer_norm_" + dtype, {"size": E, "eps": eps}, {"weight": n + ".w", "bias": n + ".b"})
            rope = PartSpec("rotary", {"head_dim": hd, "rotary_dim": hd, "theta": theta, "max_positions": P_MAX,
                                       "pairing": "half"})
            att = lambda i: PartSpec("attention", {"hidden_size": E, "num_heads": nh, "num_kv_heads": nkv, "head_dim": hd},
                                     {k: f"l{i}.{k}" for k in "qkvo"})
            ffn = lambda i: PartSpec("swiglu", {"hidden_size": E, "intermediate_size": F},
                                     {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"})
            layers = [LayerSpec("toy_parallel_" + dtype, att(0), ffn(0), ln("l0.n1"), ln("l0.unused"), rope),
                      LayerSpec("pre_norm", att(1), ffn(1), rms("l1.n1"), ln("l1.n2"), rope),
                      LayerSpec("toy_parallel_" + dtype, att(2), ffn(2), rms("l2.n1"), rms("l2.unused"), rope)]
            return ModelSpec("ToyParallelForTests_" + dtype, V, E, P_MAX,
                             PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E}, {"weight": "emb"}),
                             layers, [ScheduleEntry(i, i) for i in range(3)], ln("nf"),
                             PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "head"}))

    d = I.write_random_model(str(tmp_path / "parallel"), Cfg(), seed=8,
                             dtype=torch.float32 if dtype == "float32" else torch.bfloat16)
    w = read_weights(d)
    for n in list(w):
        if n.endswith(".b"):
            w[n] = (w[n].float() * 10 + 0.5).to(w[n].dtype)          # biases must matter
        elif w[n].dim() == 2 and n not in ("emb", "head"):
            w[n] = (w[n].float() * 4).to(w[n].dtype)                  # and so must the layers
    write_safetensors(str(tmp_path / "parallel" / "model.safetensors"), w.items())
    w = {n: t.double() for n, t in w.items()}

    def layer_norm(x, n):
        mean = x.mean(-1, keepdim=True)
        var = ((x - mean) ** 2).mean(-1, keepdim=True)
        return (x - mean) / torch.sqrt(var + eps) * w[n + ".w"] + w[n + ".b"]

    def attention(h, i, S):
        q = P.linear(h, w[f"l{i}.q"]).reshape(S, nh, hd)
        k = P.linear(h, w[f"l{i}.k"]).reshape(S, nkv, hd)
        v = P.linear(h, w[f"l{i}.v"]).reshape(S, nkv, hd)
        q = P.rope_rotate_half(q, range(S), theta, hd)
        k = P.rope_rotate_half(k, range(S), theta, hd)
        rep = nh // nkv
        k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
        return P.linear(P.causal_attention(q, k, v), w[f"l{i}.o"])

    def ffn(h, i):
        return P.swiglu_ffn(h, w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])

    def plain(ids):
        S = len(ids)
        x = P.embedding(w["emb"], ids)
        h = layer_norm(x, "l0.n1")
        x = x + attention(h, 0, S) + ffn(h, 0)
        x = x + attention(P.rms_norm(x, w["l1.n1"], eps), 1, S)
        x = x + ffn(layer_norm(x, "l1.n2"), 1)
        h = P.rms_norm(x, w["l2.n1"], eps)
        x = x + attention(h, 2, S) + ffn(h, 2)
        return P.linear(layer_norm(x, "nf"), w["head"])

    budget = 2e-5 if dtype == "float32" else 3e-2
    eng = I.Engine.from_pretrained(d, dtype=dtype, max_batch=2, max_seq_len=P_MAX)
    assert eng.runner.use_graphs
    reqs = [random_ids(n, V, 7 * n) for n in (37, 9)]
    want = [plain(r) for r in reqs]
    slots = [eng.alloc_slot(), eng.alloc_slot()]
    head = [len(r) - 4 for r in reqs]
    out = eng.step([I.StepEntry(s, r[:n], list(range(n))) for s, r, n in zip(slots, reqs, head)])
    assert rel(out[:head[0]], want[0][:head[0]]) < budget and rel(out[head[0]:], want[1][:head[1]]) < budget
    for j in range(4):                                        # the first of these is captured, the rest replayed
        out = eng.step([I.StepEntry(s, [r[n + j]], [0]) for s, r, n in zip(slots, reqs, head)])
        for b in range(2):
            assert rel(out[b], want[b][head[b] + j]) < budget, (b, j)
    # the plain computation is not blind to the toys: without the biases, or with the second
    # arrangement for the first layer, it gives other logits
    saved = w["l0.n1.b"].clone()
    w["l0.n1.b"] = torch.zeros_like(saved)
    assert rel(plain(reqs[1]), want[1]) > 10 * budget
    w["l0.n1.b"] = saved


def test_toy_embedding_and_toy_head(tmp_path):
    """The two ends as toys of the test: an embedding that scales its rows by sqrt(width), and a
    head with a bias whose logits are capped softly by a tanh.  Registered, built around one
    layer of the library's own parts, stepped whole and token by token, against a plain
    computation; generation through the entry point follows the plain argmax."""
    import inferllm_amd as I
    from inferllm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferllm_amd.kernels import ops
    from inferllm_amd.parts import Embedding, Head, register_part
    from inferllm_amd.weights import TensorWant, write_safetensors
    from tiny import random_ids, read_weights
    E, V, nh, hd, F, eps, P_MAX, theta, cap = 48, 77, 3, 16, 80, 1e-5, 64, 10000.0, 3.0

    @register_part("embedding", "toy_scaled_embedding")
    class ScaledEmbedding(Embedding):
        def __init__(self, vocab_size, hidden_size, tensors=None):
            super().__init__(tensors)
            self.V, self.E = vocab_size, hidden_size

        def shapes(self):
            return {"weight": TensorWant((self.V, self.E))}

        def load(self, tensors):
            self.weight = self._take(tensors, "weight").contiguous()

        def forward(self, ctx):
            return ops.embed(ctx.tokens, self.weight) * math.sqrt(self.E)

    @register_part("head", "toy_capped_head")
    class CappedHead(Head):
        def __init__(self, hidden_size, vocab_size, cap, tensors=None):
            super().__init__(tensors)
            self.E, self.V, self.cap = hidden_size, vocab_size, cap

        def shapes(self):
            return {"weight": TensorWant((self.V, self.E)), "bias": TensorWant((self.V,), keep_stored=True)}

        def load(self, tensors):
            self.weight = self._take(tensors, "weight").contiguous()
            self.bias = self._take(tensors, "bias").float()

        def forward(self, h, ctx):
            z = ops.linear(h, self.weight, out_dtype=torch.float32) + self.bias
            return self.cap * torch.tanh(z / self.cap)

    @register_architecture("ToyEndsForTests")
    class Cfg:
        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyEndsForTests"]}

        def to_spec(self):
            norm = lambda n: PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": n})
            rope = PartSpec("rotary", {"head_dim": hd, "rotary_dim": hd, "theta": theta, "max_positions": P_MAX,
                                       "pairing": "half"})
            layer = LayerSpec("pre_norm",
                              PartSpec("attention", {"hidden_size": E, "num_heads": nh, "num_kv_heads": nh, "head_dim": hd},
                                       {k: f"l0.{k}" for k in "qkvo"}),
                              PartSpec("swiglu", {"hidden_size": E, "intermediate_size": F},
                                       {"gate": "l0.g", "up": "l0.u", "down": "l0.d"}),
                              norm("l0.n1"), norm("l0.n2"), rope)
            return ModelSpec("ToyEndsForTests", V, E, P_MAX,
                             PartSpec("toy_scaled_embedding", {"vocab_size": V, "hidden_size": E}, {"weight": "emb"}),
                             [layer], [ScheduleEntry(0, 0)], norm("nf"),
                             PartSpec("toy_capped_head", {"hidden_size": E, "vocab_size": V, "cap": cap},
                                      {"weight": "head", "bias": "head.b"}))

    d = I.write_random_model(str(tmp_path / "ends"), Cfg(), seed=9)
    w = read_weights(d)
    w["head"] = w["head"] * 30.0                                # logits well into the cap
    w["head.b"] = w["head.b"] * 50.0
    write_safetensors(str(tmp_path / "ends" / "model.safetensors"), w.items())
    w = {n: t.double() for n, t in w.items()}

    def plain(ids):
        S = len(ids)
        x = P.embedding(w["emb"], ids) * math.sqrt(E)
        h = P.rms_norm(x, w["l0.n1"], eps)
        q, k, v = (P.linear(h, w[f"l0.{n}"]).reshape(S, nh, hd) for n in "qkv")
        q, k = P.rope_rotate_half(q, range(S), theta, hd), P.rope_rotate_half(k, range(S), theta, hd)
        x = x + P.linear(P.causal_attention(q, k, v), w["l0.o"])
        x = x + P.swiglu_ffn(P.rms_norm(x, w["l0.n2"], eps), w["l0.g"], w["l0.u"], w["l0.d"])
        z = P.linear(P.rms_norm(x, w["nf"], eps), w["head"]) + w["head.b"]
        return cap * torch.tanh(z / cap)

    eng = I.Engine.from_pretrained(d, dtype="float32", max_batch=2, max_seq_len=P_MAX)
    ids = random_ids(30, V, 4)
    want = plain(ids)
    assert float(want.abs().max()) > 0.9 * cap                 # the cap is at work
    s = eng.alloc_slot()
    out = eng.step([I.StepEntry(s, ids[:26], list(range(26)))])
    assert rel(out, want[:26]) < 2e-5
    for j in range(26, 30):
        assert rel(eng.step([I.StepEntry(s, [ids[j]], [0])])[0], want[j]) < 2e-5
    eng.free_slot(s)
    prompt = ids[:12]
    got = eng.generate([prompt], max_new_tokens=5, stop_token_ids=[])[0]
    seq = list(prompt)
    for t in got:
        logits = plain(seq)[-1]
        top2 = torch.topk(logits, 2).values
        if float(top2[0] - top2[1]) > 1e-4:                      # a near tie may go either way
            assert t == int(torch.argmax(logits))
        seq.append(t)


# ---------------------------------------------------------------- windows and steps that go on
def _windowed_architecture(name, E, V, nh, nkv, hd, F, eps, theta, windows, max_pos=1024):
    """A toy architecture whose layer i is attention with window windows[i] (None: all keys)."""
    from inferllm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture

    @register_architecture(name)
    class Cfg:
        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": [name]}

        def to_spec(self):
            norm = lambda n: PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": n})
            layers = [LayerSpec("pre_norm",
                                PartSpec("attention", {"hidden_size": E, "num_heads": nh, "num_kv_heads": nkv,
                                                       "head_dim": hd, "window": win},
                                         {k: f"l{i}.{k}" for k in "qkvo"}),
                                PartSpec("swiglu", {"hidden_size": E, "intermediate_size": F},
                                         {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                                norm(f"l{i}.n1"), norm(f"l{i}.n2"),
                                PartSpec("rotary", {"head_dim": hd, "rotary_dim": hd, "theta": theta,
                                                    "pairing": "half", "max_positions": max_pos}))
                      for i, win in enumerate(windows)]
            return ModelSpec(name, V, E, max_pos,
                             PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E}, {"weight": "emb"}),
                             layers, [ScheduleEntry(i, i) for i in range(len(windows))], norm("nf"),
                             PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "head"}))

    def plain(w, ids):
        S = len(ids)
        pos = list(range(S))
        x = P.embedding(w["emb"], ids)
        for i, win in enumerate(windows):
            h = P.rms_norm(x, w[f"l{i}.n1"], eps)
            q = P.rope_rotate_half(P.linear(h, w[f"l{i}.q"]).reshape(S, nh, hd), pos, theta)
            k = P.rope_rotate_half(P.linear(h, w[f"l{i}.k"]).reshape(S, nkv, hd), pos, theta)
            v = P.linear(h, w[f"l{i}.v"]).reshape(S, nkv, hd)
            x = x + P.linear(P.causal_attention(q, k, v, window=win), w[f"l{i}.o"])
            x = x + P.swiglu_ffn(P.rms_norm(x, w[f"l{i}.n2"], eps), w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])
        return P.linear(P.rms_norm(x, w["nf"], eps), w["head"])
    return Cfg, plain


def _scaled(d, gain):
    """The folder's matrices (not the embedding or the head) times `gain`, so that attention is
    far from uniform and a wrong or missing key moves the logits by their own size."""
    import os
    from inferllm_amd.weights import open_model_files, write_safetensors
    tensors = []
    for f in open_model_files(d):
        for n in f.names():
            t = f.read(n)
            tensors.append((n, t * gain if t.dim() == 2 and n not in ("emb", "head") else t))
        f.close()
    write_safetensors(os.path.join(d, "model.safetensors"), tensors, metadata={"format": "pt"})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("step_rows", [0, 512])
def test_a_window_model_goes_on_by_many_tokens(tmp_path, dtype, step_rows):
    """Attention with a window keeps a ring of pages.  A step stores all its keys before its rows
    read, so a sequence that goes on by more tokens than the ring holds beyond the window would
    write over keys that the step's first rows still see: the step function runs such a step in
    pieces (`step_rows=0`: a ring with 64 to 127 rows to spare), or the ring is made longer
    (`step_rows=512`).  Either way a prompt cut into steps of any lengths, a session's turns and
    `max_step_tokens` give what the whole prompt gives: layer 0 sees 70 keys, layer 1 all."""
    import inferllm_amd as I
    from tiny import random_ids, read_weights
    E, V, nh, nkv, hd, F, eps, theta, win = 64, 120, 4, 2, 16, 100, 1e-5, 10000.0, 70
    name = f"ToyWindowForTests_{dtype}_{step_rows}"
    Cfg, plain = _windowed_architecture(name, E, V, nh, nkv, hd, F, eps, theta, [win, None])
    d = I.write_random_model(str(tmp_path / "win"), Cfg(), seed=21)
    _scaled(d, 5.0)
    w = read_weights(d)
    if dtype == "bfloat16":
        w = {n: (t.to(torch.bfloat16) if t.dim() == 2 else t) for n, t in w.items()}
    tol = TOL[torch.float32 if dtype == "float32" else torch.bfloat16]
    eng = I.Engine.from_pretrained(d, dtype=dtype, max_batch=3, max_seq_len=1024, step_rows=step_rows,
                                   poison_freed=True)
    ring = next(g for g in eng.cache.groups if g.ring)
    assert ring.spec.window == win and eng.model.one_token_mixers == []
    limit = eng.cache.step_limit
    assert (64 <= limit <= 127) if step_rows == 0 else limit >= 512
    ids = random_ids(600, V, 5)
    want = plain(w, ids)
    # whole, then cut into steps: the second and third are longer than the spare rows of a short
    # ring, the fourth crosses from one piece into the next with wanted places in both
    s = eng.alloc_slot()
    got = eng.step([I.StepEntry(s, ids, list(range(len(ids))))])
    assert rel(got, want) < tol
    eng.free_slot(s)
    s, t = eng.alloc_slot(), eng.alloc_slot()
    other = random_ids(150, V, 9)
    want_other = plain(w, other)
    at = 0
    for n, picks in ((40, [39]), (200, [0, 199, 100]), (300, [299, 3]), (59, list(range(59))), (1, [0])):
        entries = [I.StepEntry(s, ids[at:at + n], picks)]
        if at == 40:
            entries.append(I.StepEntry(t, other, [149, 0]))        # a sequence that starts beside it
        out = eng.step(entries)
        for j, p in enumerate(picks):
            assert rel(out[j], want[at + p]) < tol, (at, p)
        if at == 40:
            assert rel(out[len(picks)], want_other[149]) < tol and rel(out[len(picks) + 1], want_other[0]) < tol
        at += n
    assert at == 600 and eng.cache.length(s) == 600
    eng.free_slot(s)
    eng.free_slot(t)
    eng.cache.check()
    if dtype != "float32":
        return
    # the generation loop feeds prompts in steps of 90 tokens, and a conversation goes on turn
    # after turn, with a stop token whose void step is taken back from the ring
    prompts = [ids[:230], other[:100], ids[300:420]]
    greedy = lambda p, n: [int(x) for x in _greedy(plain, w, p, n)]
    assert eng.generate(prompts, max_new_tokens=4, stop_token_ids=[], max_step_tokens=90) == \
        [greedy(p, 4) for p in prompts]
    first = greedy(ids[:150], 6)
    j = next(j for j in range(1, 6) if first[j] not in first[:j])
    with eng.session(stop_token_ids=[first[j]]) as talk:
        assert talk.say(ids[:150], max_new_tokens=6) == first[:j]
        assert talk.length == 150 + j                      # the stop token's void step was taken back
        said = list(ids[:150]) + first[:j] + list(other[:130])
        want2 = greedy(said, 3)
        if first[j] in want2:
            want2 = want2[:want2.index(first[j])]
        assert talk.say(other[:130], max_new_tokens=3) == want2
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0


def _greedy(plain, w, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(torch.argmax(plain(w, seq)[-1])))
    return seq[len(prompt):]


def test_a_toy_mixer_keeps_one_latent_row_per_token(tmp_path):
    """What a cache line keeps per token is the mixer's to say: this one keeps a single row of 12
    numbers in float32 (in a bfloat16 engine too) instead of keys and values, in the same paged
    storage with the same slots, page tables and lengths; its output is a projection of the mean
    of the rows kept so far.  Registered, built and stepped without a change to the library."""
    import inferllm_amd as I
    from inferllm_amd.cache import KVSpec, TokenTensor
    from inferllm_amd.config import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, register_architecture
    from inferllm_amd.parts import Mixer, register_part
    from inferllm_amd.weights import TensorWant
    from tiny import random_ids, read_weights
    E, R, V, eps = 40, 12, 90, 1e-5

    @register_part("mixer", "toy_latent_rows")
    class LatentRows(Mixer):
        graph_safe = False                    # reads the step's lengths on the host
        takes_continuations = True

        def __init__(self, hidden_size, rank, tensors=None):
            super().__init__(tensors)
            self.E, self.R = hidden_size, rank

        def shapes(self):
            return {"down": TensorWant((self.R, self.E)), "up": TensorWant((self.E, self.R))}

        def kv_spec(self):
            return KVSpec("full", (TokenTensor("latent", (self.R,), torch.float32),))

        def load(self, tensors):
            self.down, self.up = self._take(tensors, "down").float(), self._take(tensors, "up").float()

        def forward(self, h, ctx, line, writes_cache, position):
            kept, group = ctx.cache.token_line(line)
            rows = kept["latent"]                             # [page, row in page, R]
            c = h.float() @ self.down.t()
            pos, slot = ctx.row_pos.long(), ctx.row_slot.long()
            page = group.table[slot, pos // group.page_size].long()
            if writes_cache:
                rows[page, pos % group.page_size] = c
            out = torch.empty((h.shape[0], self.R), dtype=torch.float32, device=h.device)
            for r, (p, s) in enumerate(zip(pos.tolist(), slot.tolist())):
                js = torch.arange(p + 1, device=h.device)
                pages = group.table[s, js // group.page_size].long()
                out[r] = rows[pages, js % group.page_size].mean(dim=0)
            return (out @ self.up.t()).to(h.dtype)

    @register_architecture("ToyLatentForTests")
    class Cfg:
        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": ["ToyLatentForTests"]}

        def to_spec(self):
            norm = lambda n: PartSpec("rms_norm", {"size": E, "eps": eps}, {"weight": n})
            layers = [LayerSpec("pre_norm", PartSpec("toy_latent_rows", {"hidden_size": E, "rank": R},
                                                     {"down": f"l{i}.dn", "up": f"l{i}.up"}),
                                PartSpec("swiglu", {"hidden_size": E, "intermediate_size": 64},
                                         {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                                norm(f"l{i}.n1"), norm(f"l{i}.n2"), None) for i in range(2)]
            return ModelSpec("ToyLatentForTests", V, E, 512,
                             PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E}, {"weight": "emb"}),
                             layers, [ScheduleEntry(0, 0), ScheduleEntry(1, 1)], norm("nf"),
                             PartSpec("lm_head", {"hidden_size": E, "vocab_size": V}, {"weight": "head"}))

    def plain(w, ids):
        x = P.embedding(w["emb"], ids)
        for i in range(2):
            c = P.linear(P.rms_norm(x, w[f"l{i}.n1"], eps), w[f"l{i}.dn"])
            mean = torch.cumsum(c, 0) / torch.arange(1, len(ids) + 1, dtype=torch.float64)[:, None]
            x = x + P.linear(mean, w[f"l{i}.up"])
            x = x + P.swiglu_ffn(P.rms_norm(x, w[f"l{i}.n2"], eps), w[f"l{i}.g"], w[f"l{i}.u"], w[f"l{i}.d"])
        return P.linear(P.rms_norm(x, w["nf"], eps), w["head"])

    d = I.write_random_model(str(tmp_path / "latent"), Cfg(), seed=3)
    w = read_weights(d)
    for dtype, tol in (("float32", 2e-5), ("bfloat16", 3e-2)):
        wd = w if dtype == "float32" else {n: (t.to(torch.bfloat16) if t.dim() == 2 else t) for n, t in w.items()}
        eng = I.Engine.from_pretrained(d, dtype=dtype, max_batch=2, max_seq_len=256, poison_freed=True)
        (group,) = eng.cache.groups
        assert set(group.tensors) == {"latent"} and group.tensors["latent"].dtype == torch.float32
        assert group.tensors["latent"].shape[2:] == (64, R)
        reqs = [random_ids(n, V, n) for n in (90, 7, 70)]
        want = [plain(wd, r) for r in reqs]
        for order in ([0, 1], [2, 1]):                       # slots and pages are used again
            slots = {i: eng.alloc_slot() for i in order}
            head = {i: len(reqs[i]) - 3 for i in order}
            out = eng.step([I.StepEntry(slots[i], reqs[i][:head[i]], [head[i] - 1]) for i in order])
            for j, i in enumerate(order):
                assert rel(out[j], want[i][head[i] - 1]) < tol
            for t in range(3):
                out = eng.step([I.StepEntry(slots[i], [reqs[i][head[i] + t]], [0]) for i in order])
                for j, i in enumerate(order):
                    assert rel(out[j], want[i][head[i] + t]) < tol
            for i in order:
                eng.free_slot(slots[i])
            eng.cache.check()
        # it says it goes on by several tokens: a prompt in two steps, and generation
        s = eng.alloc_slot()
        eng.step([I.StepEntry(s, reqs[0][:50], [])])
        out = eng.step([I.StepEntry(s, reqs[0][50:], [39])])
        assert rel(out[0], want[0][89]) < tol
        eng.free_slot(s)
        if dtype == "float32":
            assert eng.generate([reqs[1]], max_new_tokens=3, stop_token_ids=[]) == [_greedy(plain, w, reqs[1], 3)]
