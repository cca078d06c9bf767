"""Tiny configurations and helpers shared by the tests.

A and B are two tiny LLaMA shapes (4 heads of 16 on 4 kv heads; 4 heads of 24 on 2 kv heads);
C adds what those two lack (another head count, tied embeddings, a head size in steps of 16 with
8-fold groups); D has the head size and grouping of the large models, E positions beyond 4,096.
They differ in every size and constant.
"""
from __future__ import annotations

import json
import os

import torch

TINY_A = {"architectures": ["LlamaForCausalLM"], "hidden_size": 64, "intermediate_size": 172,
          "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 4,
          "vocab_size": 256, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
          "max_position_embeddings": 128, "tie_word_embeddings": False,
          "bos_token_id": 1, "eos_token_id": 2}
TINY_B = {"architectures": ["LlamaForCausalLM"], "hidden_size": 96, "intermediate_size": 256,
          "num_hidden_layers": 3, "num_attention_heads": 4, "num_key_value_heads": 2,
          "head_dim": 24, "vocab_size": 320, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
          "max_position_embeddings": 256, "tie_word_embeddings": False,
          "bos_token_id": 1, "eos_token_id": [2, 3]}
TINY_C = {"architectures": ["LlamaForCausalLM"], "hidden_size": 80, "intermediate_size": 200,
          "num_hidden_layers": 1, "num_attention_heads": 8, "num_key_value_heads": 1,
          "head_dim": 32, "vocab_size": 411, "rms_norm_eps": 3e-5, "rope_theta": 25000.0,
          "max_position_embeddings": 512, "tie_word_embeddings": True,
          "bos_token_id": 0, "eos_token_id": 5}
# the head size and group layout of the large models, long positions, few parameters
TINY_D = {"architectures": ["LlamaForCausalLM"], "hidden_size": 256, "intermediate_size": 520,
          "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2,
          "head_dim": 128, "vocab_size": 1000, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
          "max_position_embeddings": 4096, "tie_word_embeddings": False,
          "bos_token_id": 1, "eos_token_id": 2}
# positions beyond 4,096: one layer of two heads of 128 on one kv head, so that the plain model
# can afford thousands of tokens
TINY_E = {"architectures": ["LlamaForCausalLM"], "hidden_size": 256, "intermediate_size": 300,
          "num_hidden_layers": 1, "num_attention_heads": 2, "num_key_value_heads": 1,
          "head_dim": 128, "vocab_size": 500, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
          "max_position_embeddings": 8192, "tie_word_embeddings": False,
          "bos_token_id": 1, "eos_token_id": 2}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E}


def make_model_dir(tmp_path, config: dict, seed: int, dtype=torch.float32, gain: float = 1.0) -> str:
    """Write a random model folder for `config` under tmp_path; returns the folder.

    gain: every matrix is multiplied by it.  The library's random weights are N(0, 0.02): with
    them queries and keys are tiny, every softmax is nearly uniform and a fault in the attention
    path (a wrong row of a projection, a wrong key) moves the logits by a per cent or two, within
    what bfloat16 is allowed.  With gain 4 the scores spread over several units and such a fault
    moves the logits by their own size."""
    import inferllm_amd as I
    from inferllm_amd.weights import open_model_files
    from inferllm_amd.weights.safetensors_io import write_safetensors
    d = os.path.join(str(tmp_path), f"model_{abs(hash(json.dumps(config, sort_keys=True))) % 10**8}_{seed}_{str(dtype)[6:]}_{gain}")
    if not os.path.isdir(d):
        I.write_random_model(d, I.config_from_dict(config), seed=seed, dtype=dtype)
        if gain != 1.0:
            tensors = []
            for f in open_model_files(d):
                for n in f.names():
                    t = f.read(n)
                    tensors.append((n, (t.float() * gain).to(t.dtype) if t.dim() == 2 else t))
                f.close()
            write_safetensors(os.path.join(d, "model.safetensors"), tensors, metadata={"format": "pt"})
    return d


def read_weights(model_dir: str):
    """All tensors of a model folder as float tensors on the CPU (for the plain model)."""
    from inferllm_amd.weights import open_model_files
    out = {}
    for f in open_model_files(model_dir):
        for n in f.names():
            out[n] = f.read(n)
        f.close()
    return out


def random_ids(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
