"""Reading and writing safetensors files by tensor name.

Format: 8 bytes little-endian header length N, N bytes of JSON
`{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}`,
then the raw little-endian data.  Files are memory-mapped; a tensor's bytes are
touched only when it is asked for, so a large checkpoint streams tensor by tensor.

The reference reads its own single-file format the same way: a header, then
records found by name, data read on demand (src/core/graph.cpp:270-333,
src/core/tensor.cpp:78-121, src/file.cpp:7-61).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8,
    "U8": torch.uint8, "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class PinnedStage:
    """Two pinned host buffers used in turn for copies to the device."""

    def __init__(self, nbytes: int = 64 << 20):
        self.nbytes = nbytes
        self._bufs = [torch.empty(nbytes, dtype=torch.uint8, pin_memory=True) for _ in range(2)]
        self._events = [None, None]
        self._i = 1

    def next(self) -> torch.Tensor:
        self._i ^= 1
        if self._events[self._i] is not None:
            self._events[self._i].synchronize()
        return self._bufs[self._i]

    def sent(self) -> None:
        ev = torch.cuda.Event()
        ev.record()
        self._events[self._i] = ev

    def finish(self) -> None:
        for ev in self._events:
            if ev is not None:
                ev.synchronize()


class SafetensorsFile:
    """One memory-mapped file: `.entries` maps names to (dtype string, shape)."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors file")
        self._f = open(path, "rb")
        (n,) = struct.unpack("<Q", self._f.read(8))
        if n <= 0 or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._f.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON ({e})") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._data_start = 8 + n
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.entries: Dict[str, Tuple[str, Tuple[int, ...]]] = {}
        self._offsets: Dict[str, Tuple[int, int]] = {}
        for name, e in header.items():
            dt, shape = e.get("dtype"), tuple(int(s) for s in e.get("shape", ()))
            b, t = (int(v) for v in e.get("data_offsets", (0, 0)))
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name!r} has unsupported dtype {dt!r}")
            count = 1
            for s in shape:
                count *= s
            nbytes = count * torch.empty((), dtype=_DTYPES[dt]).element_size()
            if t - b != nbytes or b < 0 or self._data_start + t > size:
                raise SafetensorsError(
                    f"{path}: tensor {name!r} ({dt}, {list(shape)}) needs {nbytes} bytes "
                    f"but its offsets give {t - b}")
            self.entries[name] = (dt, shape)
            self._offsets[name] = (b, t)

    def names(self) -> List[str]:
        return list(self.entries)

    def read(self, name: str) -> torch.Tensor:
        """The tensor as stored (a copy that owns its memory)."""
        dt, shape = self.entries[name]
        b, t = self._offsets[name]
        dtype = _DTYPES[dt]
        if t == b:
            return torch.empty(shape, dtype=dtype)
        raw = bytearray(self._map[self._data_start + b:self._data_start + t])   # one copy, owned
        return torch.frombuffer(raw, dtype=dtype).reshape(shape)

    def read_to_device(self, name: str, device, stage: "PinnedStage") -> torch.Tensor:
        """The tensor as stored, on a GPU: the file's bytes go through two pinned host buffers
        in turn, one being filled from the file while the other is copied to the device."""
        dt, shape = self.entries[name]
        b, t = self._offsets[name]
        out = torch.empty(shape, dtype=_DTYPES[dt], device=device)
        if t == b:
            return out
        flat = out.view(-1).view(torch.uint8)
        pos, end, done = self._data_start + b, self._data_start + t, 0
        while pos < end:
            n = min(stage.nbytes, end - pos)
            buf = stage.next()                      # waits for the copy that last used it
            got = os.preadv(self._f.fileno(), [memoryview(buf.numpy())[:n]], pos)
            if got != n:
                raise SafetensorsError(f"{self.path}: short read of tensor {name!r}")
            flat[done:done + n].copy_(buf[:n], non_blocking=True)
            stage.sent()
            pos += n
            done += n
        return out

    def close(self) -> None:
        try:
            self._map.close()
        except BufferError:
            pass
        self._f.close()


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]],
                      metadata: Dict[str, str] | None = None) -> None:
    """Write (name, tensor) pairs; tensors are taken to the CPU one at a time."""
    offset = 0
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    data_tmp = path + ".data.tmp"
    with open(data_tmp, "wb") as data:
        for name, t in tensors:
            if name in header:
                raise SafetensorsError(f"duplicate tensor name {name!r}")
            if t.dtype not in _NAMES:
                raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
            t = t.detach().to("cpu").contiguous()
            nbytes = t.numel() * t.element_size()
            header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                            "data_offsets": [offset, offset + nbytes]}
            offset += nbytes
            if nbytes:
                raw = t.to(torch.uint8) if t.dtype == torch.bool else t.reshape(-1).view(torch.uint8)
                data.write(raw.numpy().tobytes())
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f, open(data_tmp, "rb") as data:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        while True:
            chunk = data.read(1 << 26)
            if not chunk:
                break
            f.write(chunk)
    os.remove(data_tmp)
    os.replace(tmp, path)


def open_model_files(model_dir: str) -> List[SafetensorsFile]:
    """`model.safetensors`, or the shards that `model.safetensors.index.json` names."""
    single = os.path.join(model_dir, "model.safetensors")
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(single):
        return [SafetensorsFile(single)]
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            weight_map = json.load(f).get("weight_map", {})
        shards = sorted(set(weight_map.values()))
        if not shards:
            raise SafetensorsError(f"{index}: empty weight_map")
        return [SafetensorsFile(os.path.join(model_dir, s)) for s in shards]
    raise SafetensorsError(f"no model.safetensors (or model.safetensors.index.json) in {model_dir!r}")
