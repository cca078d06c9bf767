"""Seeded random weights: a model folder (config.json, model.safetensors) from a
configuration and a seed, or the same tensors handed over in memory.

Each tensor has a generator of its own, seeded by (seed, tensor name), so a
tensor's values depend neither on the order of the tensors nor on which others
exist.  Linear and embedding weights are N(0, 0.02), norm weights 1 + N(0, 0.01),
drawn in float32 and then rounded to the stored dtype.  The reference has random
weights in its op tests only (test/checker.cpp:138-151: normal values from a
seeded std::mt19937).
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict, Iterator, Tuple

import torch

from .loader import TensorWant
from .safetensors_io import write_safetensors

LINEAR_STD = 0.02
NORM_STD = 0.01


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{int(seed)}:{name}".encode("utf-8")).digest()
    return int.from_bytes(h[:8], "little") & ((1 << 63) - 1)


def random_tensor(seed: int, name: str, want: TensorWant, dtype: torch.dtype,
                  device: torch.device | str = "cpu") -> torch.Tensor:
    """One tensor; values are a function of (seed, name, shape, kind of device)."""
    g = torch.Generator(device=device)
    g.manual_seed(_tensor_seed(seed, name))
    if want.kind == "int":
        raise ValueError(f"no random rule for the integer table {name!r}")
    t = torch.randn(want.shape, generator=g, dtype=torch.float32, device=device)
    if want.init == "ones_normal":
        t.mul_(NORM_STD).add_(1.0)
    elif want.init == "normal":
        t.mul_(LINEAR_STD)
    else:
        raise ValueError(f"unknown random rule {want.init!r} for {name!r}")
    return t.to(dtype)


def random_tensors(expected: Dict[str, TensorWant], seed: int, dtype: torch.dtype,
                   device: torch.device | str = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    for name, want in expected.items():
        if want.optional:
            continue
        yield name, random_tensor(seed, name, want, dtype, device)


def write_random_model(model_dir: str, config, seed: int, dtype: torch.dtype = torch.float32) -> str:
    """Write `config.json` and `model.safetensors` for a typed configuration; returns the folder."""
    from ..engine.model import expected_tensors  # late: the model layer imports this package
    os.makedirs(model_dir, exist_ok=True)
    d = config.to_dict()
    d["torch_dtype"] = {torch.float32: "float32", torch.bfloat16: "bfloat16",
                        torch.float16: "float16"}[dtype]
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(d, f, indent=1)
    expected = expected_tensors(config.to_spec())
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      random_tensors(expected, seed, dtype),
                      metadata={"format": "pt", "seed": str(seed)})
    return model_dir
