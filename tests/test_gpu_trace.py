"""Trace replay through `bin/trace_run` as a user runs it (a child process fed over a
pipe): the same requests whole, with the last 32 tokens one by one, and in batches of
unequal lengths whose shorter requests end earlier, in float32 and in bfloat16, all
against the plain implementation."""
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
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BUDGET = {"float32": 2e-5, "bfloat16": 3e-2}
STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def replay(model_dir, dtype, out_dir, max_tokens, steps):
    """Feed `steps` one at a time, waiting for each `done`; returns {step: logits array}."""
    p = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
                          "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)],
                         stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in steps:
            p.stdin.write(json.dumps(s) + "\n")
            p.stdin.flush()
            line = p.stdout.readline().strip()
            assert line == f"done {s['step']}", f"step {s['step']}: got {line!r}"
        p.stdin.close()
        assert p.wait(timeout=60) == 0
    finally:
        if p.poll() is None:
            p.kill()
    out = {}
    for s in steps:
        f = os.path.join(out_dir, f"{s['step']}.f32")
        n = sum(len(e.get("want", [])) for e in s["entries"])
        assert os.path.exists(f) == (n > 0)
        if n:
            out[s["step"]] = np.fromfile(f, dtype="<f4").reshape(n, -1)
    return out


def worst(got, want):
    return float(np.abs(got.astype(np.float64) - want.numpy()).max() / want.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_three_schedules_agree_with_the_plain_model(tmp_path, name, dtype):
    config = CONFIGS[name]
    d = make_model_dir(tmp_path, config, seed=13, dtype=STORE[dtype], gain=4.0)
    w = read_weights(d)
    lens = [40, 70, 33, 100, 36]
    reqs = [random_ids(n, config["vocab_size"], 100 + i) for i, n in enumerate(lens)]
    plain = [plain_llama.forward_logits(config, w, r) for r in reqs]
    steps, expect = [], {}
    n = 0
    # 1. whole, each alone
    for i, r in enumerate(reqs):
        steps.append({"step": n, "entries": [{"id": f"w{i}", "tokens": r, "want": list(range(len(r)))}],
                      "end": [f"w{i}"]})
        expect[n] = plain[i]; n += 1
    # 2. the last 32 tokens one by one
    for i, r in enumerate(reqs):
        head = len(r) - 32
        steps.append({"step": n, "entries": [{"id": f"t{i}", "tokens": r[:head], "want": list(range(head))}], "end": []})
        expect[n] = plain[i][:head]; n += 1
        for j in range(head, len(r)):
            steps.append({"step": n, "entries": [{"id": f"t{i}", "tokens": [r[j]], "want": [0]}],
                          "end": [f"t{i}"] if j == len(r) - 1 else []})
            expect[n] = plain[i][j:j + 1]; n += 1
    # 3. batches of unequal lengths; the shorter end earlier; ids are reused, so are slots
    for batch in ([0, 1, 2], [3, 4], [2, 0, 3]):
        prompt = {i: len(reqs[i]) - 3 - 2 * k for k, i in enumerate(batch)}
        steps.append({"step": n, "entries": [{"id": f"b{i}", "tokens": reqs[i][:prompt[i]], "want": [0, prompt[i] - 1]}
                                             for i in batch], "end": []})
        expect[n] = torch.cat([plain[i][[0, prompt[i] - 1]] for i in batch]); n += 1
        at = dict(prompt)
        live = list(batch)
        while live:
            ends = [i for i in live if at[i] == len(reqs[i]) - 1]
            steps.append({"step": n, "entries": [{"id": f"b{i}", "tokens": [reqs[i][at[i]]], "want": [0]} for i in live],
                          "end": [f"b{i}" for i in ends]})
            expect[n] = torch.cat([plain[i][at[i]:at[i] + 1] for i in live]); n += 1
            for i in live:
                at[i] += 1
            live = [i for i in live if i not in ends]
    # room: the largest batch holds 128 + 128 + 64 tokens in pages of 64
    got = replay(d, dtype, str(tmp_path / "out"), 320, steps)
    bad = [(s, worst(got[s], expect[s])) for s in sorted(expect) if worst(got[s], expect[s]) >= BUDGET[dtype]]
    assert not bad, f"first wrong step: {bad[0]}"


def test_a_step_that_wants_nothing_writes_nothing_and_bad_input_fails(tmp_path):
    config = CONFIGS["A"]
    d = make_model_dir(tmp_path, config, seed=1)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [4], "want": [0]}], "end": ["a"]}]
    got = replay(d, "float32", str(tmp_path / "o"), 64, steps)
    assert list(got) == [1] and got[1].shape == (1, 256)
    w = read_weights(d)
    assert worst(got[1], plain_llama.forward_logits(config, w, [1, 2, 3, 4])[3:]) < 2e-5
    # more tokens than --max-tokens allows: the program fails rather than computing garbage
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32",
                        "--out", str(tmp_path / "o2"), "--max-tokens", "64"],
                       input=json.dumps({"step": 0, "entries": [{"id": "a", "tokens": list(range(65)), "want": [0]}],
                                         "end": []}) + "\n", capture_output=True, text=True)
    assert p.returncode != 0 and "cache full" in p.stderr
