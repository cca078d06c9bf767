"""Configurations off the beaten sizes, end to end against the plain model: head sizes that are
no power of two or no multiple of 16, widths and feed-forward sizes that are no multiple of 8 or
32, odd vocabularies, a width that is not heads x head size, tied embeddings, groups of 3, 4 and 7.
Prompts of unequal lengths in one step, then three tokens each, in 32-bit and in bfloat16, with and
without the decode copies of the matrices."""
import pytest
import torch

import plain_llama
from tiny import make_model_dir, random_ids, read_weights

pytestmark = pytest.mark.gpu

BASE = {"architectures": ["LlamaForCausalLM"], "rms_norm_eps": 2e-5, "rope_theta": 12345.0,
        "max_position_embeddings": 300, "tie_word_embeddings": False, "bos_token_id": 1,
        "eos_token_id": 2}
CASES = [
    dict(hidden_size=120, intermediate_size=130, num_hidden_layers=2, num_attention_heads=3,
         num_key_value_heads=3, head_dim=48, vocab_size=777),
    dict(hidden_size=72, intermediate_size=99, num_hidden_layers=1, num_attention_heads=6,
         num_key_value_heads=2, head_dim=12, vocab_size=1001),
    dict(hidden_size=224, intermediate_size=608, num_hidden_layers=2, num_attention_heads=7,
         num_key_value_heads=7, head_dim=32, vocab_size=50),
    dict(hidden_size=320, intermediate_size=96, num_hidden_layers=1, num_attention_heads=20,
         num_key_value_heads=5, head_dim=16, vocab_size=3000, tie_word_embeddings=True),
    dict(hidden_size=192, intermediate_size=500, num_hidden_layers=1, num_attention_heads=3,
         num_key_value_heads=1, head_dim=64, vocab_size=129),
]
BUDGET = {"float32": 2e-5, "bfloat16": 3e-2}
STORE = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.mark.parametrize("copies", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_odd_configuration_equals_plain(tmp_path_factory, case, dtype, copies):
    import inferllm_amd as I
    from inferllm_amd import StepEntry
    config = dict(BASE, **CASES[case])
    d = make_model_dir(tmp_path_factory.getbasetemp(), config, seed=case, dtype=STORE[dtype], gain=4.0)
    w = read_weights(d)
    eng = I.Engine.from_pretrained(d, dtype=dtype, device="cuda:0", max_batch=8,
                                   decode_copies=copies, poison_freed=True)
    reqs = [random_ids(n + 3, config["vocab_size"], 5 * case + n) for n in (1, 9, 70, 33, 17, 130)]
    slots = [eng.alloc_slot() for _ in reqs]
    got = [[] for _ in reqs]
    out = eng.step([StepEntry(s, r[:-3], list(range(len(r) - 3))) for s, r in zip(slots, reqs)])
    at = 0
    for i, r in enumerate(reqs):
        got[i].append(out[at:at + len(r) - 3].clone())
        at += len(r) - 3
    for t in (3, 2, 1):
        out = eng.step([StepEntry(s, [r[-t]], [0]) for s, r in zip(slots, reqs)])
        for i in range(len(reqs)):
            got[i].append(out[i:i + 1].clone())
    for i, r in enumerate(reqs):
        want = plain_llama.forward_logits(config, w, r)
        worst = float((torch.cat(got[i]).double().cpu() - want).abs().max() / want.abs().max())
        assert worst < BUDGET[dtype], (i, worst)
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()
