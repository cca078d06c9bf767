"""What stands behind the engine's numbers: folders stored in float16 and float32 run in a
bfloat16 engine on the serving kernels, random weights drawn on the device are what the plain
model computes with, the float32 path at the real layer sizes, and the same request gives the
same bits in another process."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama
from tiny import CONFIGS, make_model_dir, random_ids, read_weights

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUDGET = {"float32": 2e-5, "bfloat16": 3e-2}

REAL = {"architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "intermediate_size": 11008,
        "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 32,
        "vocab_size": 32000, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
        "max_position_embeddings": 512, "tie_word_embeddings": False,
        "bos_token_id": 1, "eos_token_id": 2}


def three_schedules(eng, reqs, tail):
    """Logits [len, vocab] of every request under three schedules: whole; the last `tail` tokens
    one by one; all requests as one batch of unequal prompts whose shorter ones end earlier."""
    from inferllm_amd import StepEntry
    out = {"whole": [], "tail": [], "batch": []}
    for r in reqs:
        s = eng.alloc_slot()
        out["whole"].append(eng.step([StepEntry(s, r, list(range(len(r))))]).clone())
        eng.free_slot(s)
    for r in reqs:
        s = eng.alloc_slot()
        head = len(r) - tail
        got = [eng.step([StepEntry(s, r[:head], list(range(head)))]).clone()]
        for t in r[head:]:
            got.append(eng.step([StepEntry(s, [t], [0])]).clone())
        out["tail"].append(torch.cat(got))
        eng.free_slot(s)
    slots = [eng.alloc_slot() for _ in reqs]
    prompt = [max(1, len(r) - 3 - 2 * i) for i, r in enumerate(reqs)]
    got = [[] for _ in reqs]
    logits = eng.step([StepEntry(s, r[:p], list(range(p))) for s, r, p in zip(slots, reqs, prompt)])
    at = 0
    for i, p in enumerate(prompt):
        got[i].append(logits[at:at + p].clone())
        at += p
    pos = list(prompt)
    live = [i for i in range(len(reqs)) if pos[i] < len(reqs[i])]
    while live:
        logits = eng.step([StepEntry(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
        for j, i in enumerate(live):
            got[i].append(logits[j:j + 1].clone())
            pos[i] += 1
        for i in [i for i in live if pos[i] == len(reqs[i])]:
            eng.free_slot(slots[i])
        live = [i for i in live if pos[i] < len(reqs[i])]
    out["batch"] = [torch.cat(g) for g in got]
    eng.cache.check()
    assert eng.cache.slots.n_held() == 0
    return out


def check_schedules(got, want, budget):
    for name, per_req in got.items():
        for i, (g, w) in enumerate(zip(per_req, want)):
            per_pos = (g.double().cpu() - w).abs().max(dim=1).values / w.abs().max()
            assert float(per_pos.max()) < budget, \
                f"{name}, request {i}: first bad position {int((per_pos >= budget).nonzero()[0])} of {len(w)}"


def rounded(w):
    """The plain model's weights for a bfloat16 engine: matrices rounded to bfloat16 (to nearest
    even, what the loader does), norm weights as stored."""
    return {n: (t.float().to(torch.bfloat16) if t.dim() == 2 else t) for n, t in w.items()}


@pytest.mark.parametrize("stored", [torch.float16, torch.float32])
@pytest.mark.parametrize("name", ["B", "real"])
def test_float16_and_float32_folders_in_a_bfloat16_engine(tmp_path, monkeypatch, name, stored):
    """LLaMA-2 ships in float16.  Such a folder (and a float32 one) loads into a bfloat16 engine
    with its matrices rounded to bfloat16 on the way, gets decode copies like a bfloat16 folder,
    and no product falls to the float32 multiply-add kernel."""
    import inferllm_amd as I
    from inferllm_amd.kernels import ops
    if name == "real" and stored == torch.float32:
        pytest.skip("the float16 folder covers the real sizes; float32 would only double the file")
    config = CONFIGS["B"] if name == "B" else REAL
    d = make_model_dir(tmp_path, config, seed=21, dtype=stored, gain=4.0 if name == "B" else 2.0)
    w = rounded(read_weights(d))
    eng = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=4, poison_freed=True)
    assert eng.decode_copies is True
    for layer in eng.model.layers:
        for m in (layer.mixer.w_qkv, layer.mixer.w_o, layer.feed_forward.w_gate_up, layer.feed_forward.w_down):
            assert m.dtype == torch.bfloat16
            if name == "real":                      # decode copies as for a bfloat16 folder
                assert isinstance(m, ops.Weight) and m.tiled is not None
        assert layer.mixer_norm.weight.dtype == torch.float32        # norm weights keep their precision
    slow = []
    for fn in ("gemm_generic", "gemv_rows_f32"):
        real = getattr(ops, fn)
        monkeypatch.setattr(ops, fn, lambda *a, _f=fn, _r=real: slow.append(_f) or _r(*a))
    lens = [40, 70, 33] if name == "B" else [40, 23, 37]
    reqs = [random_ids(n, config["vocab_size"], 50 + i) for i, n in enumerate(lens)]
    want = [plain_llama.forward_logits(config, w, r) for r in reqs]
    check_schedules(three_schedules(eng, reqs, tail=16), want, BUDGET["bfloat16"])
    assert not slow, f"products fell to the float32 kernel: {sorted(set(slow))}"


def test_keep_stored_keeps_32_bits_and_warns(tmp_path):
    import inferllm_amd as I
    d = make_model_dir(tmp_path, CONFIGS["A"], seed=3, dtype=torch.float16, gain=4.0)
    with pytest.warns(UserWarning, match="stay float32"):
        eng = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, keep_stored=True)
    assert eng.model.layers[0].feed_forward.w_down.dtype == torch.float32
    w = read_weights(d)
    ids = random_ids(20, 256, 1)
    s = eng.alloc_slot()
    got = eng.step([I.StepEntry(s, ids, list(range(20)))])
    want = plain_llama.forward_logits(CONFIGS["A"], w, ids)
    assert float((got.double().cpu() - want).abs().max() / want.abs().max()) < BUDGET["bfloat16"]


def engine_tensors(eng):
    """The engine's weights under their checkpoint names, read back from its parts."""
    spec = eng.spec
    out = {}
    from inferllm_amd.kernels import ops
    plain = ops.plain_weight
    for ls, layer in zip(spec.layers, eng.model.layers):
        m, f = layer.mixer, layer.feed_forward
        qkv = plain(m.w_qkv)
        nq, nk = m.nh * m.hd, m.nkv * m.hd
        out[ls.mixer.tensors["q"]] = qkv[:nq]
        out[ls.mixer.tensors["k"]] = qkv[nq:nq + nk]
        out[ls.mixer.tensors["v"]] = qkv[nq + nk:]
        out[ls.mixer.tensors["o"]] = plain(m.w_o)
        gu = plain(f.w_gate_up)
        out[ls.feed_forward.tensors["gate"]] = gu[:f.F]
        out[ls.feed_forward.tensors["up"]] = gu[f.F:]
        out[ls.feed_forward.tensors["down"]] = plain(f.w_down)
        out[ls.mixer_norm.tensors["weight"]] = layer.mixer_norm.weight
        out[ls.feed_forward_norm.tensors["weight"]] = layer.feed_forward_norm.weight
    out[spec.embedding.tensors["weight"]] = eng.model.embedding.weight
    out[spec.final_norm.tensors["weight"]] = eng.model.final_norm.weight
    out[spec.head.tensors["weight"]] = plain(eng.model.head.weight)
    return {n: t.detach().cpu() for n, t in out.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_random_weights_drawn_on_the_device(name, dtype):
    """`Engine.from_random` (what the benchmark and `chat --random` run on): the tensors the
    engine holds, fed to the plain model, give the engine's logits and greedy tokens; the same
    seed gives the same tensors, another seed others; values have the documented spread."""
    import inferllm_amd as I
    config = CONFIGS[name]
    eng = I.Engine.from_random(config, seed=5, dtype=dtype, device=DEV, max_batch=4, poison_freed=True)
    w = engine_tensors(eng)
    again = engine_tensors(I.Engine.from_random(config, seed=5, dtype=dtype, device=DEV))
    other = engine_tensors(I.Engine.from_random(config, seed=6, dtype=dtype, device=DEV))
    assert set(w) == set(again) and all(torch.equal(w[n], again[n]) for n in w)
    assert all(not torch.equal(w[n], other[n]) for n in w)
    for n, t in w.items():
        t = t.float()
        if t.dim() == 2:
            assert abs(float(t.mean())) < 2e-3 and 0.018 < float(t.std()) < 0.022, n     # N(0, 0.02)
        else:
            assert abs(float(t.mean()) - 1) < 5e-3 and 0.005 < float(t.std()) < 0.015, n  # 1 + N(0, 0.01)
    reqs = [random_ids(n, config["vocab_size"], 70 + i) for i, n in enumerate([40, 9, 65])]
    want = [plain_llama.forward_logits(config, w, r) for r in reqs]
    check_schedules(three_schedules(eng, reqs, tail=8), want, BUDGET[dtype])
    if dtype == "float32":
        got = eng.generate([r[:6] for r in reqs], max_new_tokens=8, stop_token_ids=[])
        assert got == [plain_llama.generate_greedy(config, w, r[:6], 8) for r in reqs]


def test_chat_with_random_weights_prints_the_plain_models_tokens(tmp_path, capsys):
    """`chat --random CONFIG --weights-seed N`: the tokens printed are the plain model's greedy
    tokens on the same tensors."""
    import inferllm_amd as I
    from inferllm_amd.cli.chat import main
    config = CONFIGS["A"]
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(config))
    rc = main(["--random", str(cfg_file), "--weights-seed", "9", "-d", "float32", "--temp", "0",
               "--prompt-ids", "1,5,9,200", "-n", "7", "--stop-ids", "255"])
    assert rc == 0
    printed = [int(t) for t in capsys.readouterr().out.split()]
    w = engine_tensors(I.Engine.from_random(config, seed=9, dtype="float32", device=DEV))
    want = plain_llama.generate_greedy(config, w, [1, 5, 9, 200], 7)
    if 255 in want:
        want = want[:want.index(255)]
    assert printed == want


@pytest.mark.parametrize("nkv,ffn", [(32, 11008), (8, 14336)])
def test_real_layer_sizes_in_float32(tmp_path, nkv, ffn):
    """Two layers of the LLaMA-2-7B and LLaMA-3-8B sizes on the true 32-bit path under all three
    schedules: the float32 products over 4096 and 11008 / 14336, the float32 attention at head
    size 128 with and without grouped heads, against the plain model within the float32 budget."""
    import inferllm_amd as I
    config = dict(REAL, intermediate_size=ffn, num_key_value_heads=nkv)
    d = make_model_dir(tmp_path, config, seed=11, dtype=torch.float32, gain=2.0)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype="float32", device=DEV, max_batch=4, poison_freed=True)
    reqs = [random_ids(n, config["vocab_size"], 90 + i) for i, n in enumerate([37, 20, 49])]
    want = [plain_llama.forward_logits(config, w, r) for r in reqs]
    check_schedules(three_schedules(eng, reqs, tail=16), want, BUDGET["float32"])


def _replay(model_dir, out_dir, steps):
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
                        "--dtype", "bfloat16", "--out", out_dir, "--max-tokens", "4096"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    return {s["step"]: np.fromfile(os.path.join(out_dir, f"{s['step']}.f32"), dtype="<f4") for s in steps}


def test_two_processes_give_the_same_bfloat16_bits(tmp_path):
    """Which kernel a bfloat16 product takes is a table entry by shape, never a measurement: the
    same trace replayed by two fresh processes gives bit-equal logits (real layer sizes, so that
    every table entry of the 7B shapes is in play: a prompt of 1,100 tokens, one of 100, decode
    steps of 2 and of 13 rows)."""
    d = make_model_dir(tmp_path, dict(REAL, max_position_embeddings=2048), seed=4, dtype=torch.bfloat16,
                       gain=2.0)
    vocab = REAL["vocab_size"]
    long, short = random_ids(1100, vocab, 1), random_ids(100, vocab, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": long, "want": [0, 1099]},
                                     {"id": "b", "tokens": short, "want": [99]}], "end": []}]
    for t in range(3):
        steps.append({"step": 1 + t, "entries": [{"id": "a", "tokens": [7 + t], "want": [0]},
                                                 {"id": "b", "tokens": [9 + t], "want": [0]}],
                      "end": ["a", "b"] if t == 2 else []})
    many = [random_ids(5 + i, vocab, 10 + i) for i in range(13)]
    steps.append({"step": 4, "entries": [{"id": f"m{i}", "tokens": r, "want": [len(r) - 1]}
                                         for i, r in enumerate(many)], "end": []})
    steps.append({"step": 5, "entries": [{"id": f"m{i}", "tokens": [3 + i], "want": [0]} for i in range(13)],
                  "end": [f"m{i}" for i in range(13)]})
    first = _replay(d, str(tmp_path / "o1"), steps)
    second = _replay(d, str(tmp_path / "o2"), steps)
    for s in first:
        assert np.isfinite(first[s]).all()
        assert first[s].tobytes() == second[s].tobytes(), f"step {s} differs between two processes"


def test_a_pinned_plan_gives_the_same_bits_and_tuning_happens_at_construction(tmp_path):
    """`Engine(tune=True)` times the thin matrices while it is built (not in the first request)
    and keeps what won in `engine.plan`; an engine given that plan takes the same kernels without
    a stopwatch and gives bit-equal logits."""
    import inferllm_amd as I
    from inferllm_amd.kernels import ops
    config = dict(REAL, num_hidden_layers=1)
    d = make_model_dir(tmp_path, config, seed=8, dtype=torch.bfloat16, gain=2.0)
    tuned = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=16, tune=True)
    shape = (config["hidden_size"], config["intermediate_size"])
    assert tuned.plan.planes_from.get(shape) in (1, 5, 9, 13, 17)      # there before any step
    reqs = [random_ids(4 + i, config["vocab_size"], 30 + i) for i in range(12)]

    def run(eng):
        slots = [eng.alloc_slot() for _ in reqs]
        a = eng.step([I.StepEntry(s, r, [len(r) - 1]) for s, r in zip(slots, reqs)]).clone()
        b = eng.step([I.StepEntry(s, [5], [0]) for s in slots]).clone()
        for s in slots:
            eng.free_slot(s)
        return a, b
    want = run(tuned)
    pinned = I.Engine.from_pretrained(d, dtype="bfloat16", device=DEV, max_batch=16,
                                      plan=json.loads(json.dumps(tuned.plan.to_dict())))
    assert not pinned.plan.measure and pinned.plan == tuned.plan
    timed = []
    real = ops.measure_planes_from
    ops.measure_planes_from = lambda w: timed.append(1) or real(w)
    try:
        got = run(pinned)
    finally:
        ops.measure_planes_from = real
    assert not timed
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
