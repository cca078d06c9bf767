"""Weights by tensor name, checked as a whole before anything is computed.

The model says which tensors it wants (`expected`: name -> `TensorWant`); the
loader finds each by name in the folder's safetensors files, checks all of them
and raises ONE error that lists every missing tensor, every unexpected tensor
and every wrong shape.  The reference does the name lookup while it scans the
file (src/core/graph.cpp:285-331), skips unknown names with a log line
(:311-317), asserts on a wrong element count (:322-326) and never notices a
missing weight; here all three are errors.

Precision in memory.  The reference gives every tensor the runtime type that the
file's type code names (src/core/graph.cpp:216-231).  Here a floating tensor becomes
the engine's dtype as it is loaded: in a bfloat16 engine float16 and float32
matrices are rounded to bfloat16 (to nearest, ties to even, on the device), so that
a checkpoint stored in float16 runs on the same kernels as one stored in bfloat16.
Tensors that the model marks `keep_stored` (norm weights and the like: small, and
read by kernels that take either type) keep what the file holds: bfloat16 stays
bfloat16, 32-bit stays 32-bit, float16 is widened to float32 (exact).  With
`keep_stored=True` for the whole load every tensor is treated so.  Integer tables
become int32.  An engine that runs in float32 widens every floating tensor to
float32 (exact for all three stored types).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, Tuple

import torch

from .safetensors_io import PinnedStage, SafetensorsFile, open_model_files


class WeightsError(ValueError):
    """Raised once per load with everything that is wrong with the checkpoint."""

    def __init__(self, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = ["checkpoint does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name} is {list(got)}, the model needs {list(want)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  wrong dtype: {name} is stored as {got}")
        super().__init__("\n".join(lines))


@dataclass
class TensorWant:
    """What the model needs of one checkpoint tensor."""
    shape: Tuple[int, ...]
    kind: str = "float"          # "float" or "int"
    init: str = "normal"         # random-weights rule: "normal" N(0, s) or "ones_normal" 1 + N(0, s)
    optional: bool = False       # absent is fine (e.g. a head tied to the embedding)
    keep_stored: bool = False    # keeps the file's precision in a bfloat16 engine (norm weights)


_FLOATS = {"F64", "F32", "F16", "BF16"}
_INTS = {"I64", "I32", "I16", "I8", "U8"}


def check_names(expected: Dict[str, TensorWant],
                stored: Dict[str, Tuple[str, Tuple[int, ...]]],
                ignored_suffixes: Iterable[str] = ()) -> None:
    """Raise `WeightsError` unless `stored` (name -> (dtype string, shape)) fits `expected`."""
    ignored = tuple(ignored_suffixes)
    missing = [n for n, w in expected.items() if n not in stored and not w.optional]
    unexpected = [n for n in stored if n not in expected and not (ignored and n.endswith(ignored))]
    wrong_shape, wrong_dtype = [], []
    for n, w in expected.items():
        if n in stored:
            dt, shape = stored[n]
            if tuple(shape) != tuple(w.shape):
                wrong_shape.append((n, tuple(w.shape), tuple(shape)))
            if (w.kind == "float" and dt not in _FLOATS) or (w.kind == "int" and dt not in _INTS):
                wrong_dtype.append((n, dt))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightsError(sorted(missing), sorted(unexpected), wrong_shape, wrong_dtype)


def kept_dtype(stored: torch.dtype, kind: str, engine_dtype: torch.dtype,
               keep_stored: bool = False) -> torch.dtype:
    """The dtype a stored tensor has in memory (see the module text)."""
    if kind == "int":
        return torch.int32
    if engine_dtype == torch.float32:
        return torch.float32
    if stored == torch.bfloat16 or not keep_stored:
        return torch.bfloat16
    return torch.float32


def load_named_tensors(model_dir: str, expected: Dict[str, TensorWant], engine_dtype: torch.dtype,
                       device: torch.device | str,
                       ignored_suffixes: Iterable[str] = (),
                       keep_stored: bool = False) -> Dict[str, torch.Tensor]:
    """All expected tensors that the folder holds, on `device`, after the whole-folder check.
    `keep_stored`: no floating tensor is rounded to the engine's dtype (see the module text)."""
    files: List[SafetensorsFile] = open_model_files(model_dir)
    try:
        where: Dict[str, SafetensorsFile] = {}
        stored: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        for f in files:
            for n, e in f.entries.items():
                where[n] = f
                stored[n] = e
        check_names(expected, stored, ignored_suffixes)
        out: Dict[str, torch.Tensor] = {}
        on_gpu = torch.device(device).type == "cuda"
        stage = PinnedStage() if on_gpu else None
        for n, w in expected.items():
            if n not in where:
                continue
            if on_gpu and w.kind != "int":
                with torch.cuda.device(device):
                    t = where[n].read_to_device(n, device, stage)
            else:
                t = where[n].read(n)
                if w.kind == "int" and t.numel() and (int(t.max()) > 2**31 - 1 or int(t.min()) < -2**31):
                    raise WeightsError([], [], [], [(n, "integers beyond int32")])
            out[n] = t.to(device=device, dtype=kept_dtype(t.dtype, w.kind, engine_dtype,
                                                          keep_stored or w.keep_stored))
        if stage is not None:
            stage.finish()
        return out
    finally:
        for f in files:
            f.close()
