"""A reader and a writer for the safetensors container: `[u64 LE header length][JSON][data]`.

The reader maps the file and hands out tensors by name without copying; it checks what the
reference's reader checks before it trusts a header (src/safetensors.rs:177-296): the length
fits the file and is at most 100 MB, the header is a JSON object, every tensor has a known
dtype, at most 4 dimensions and a byte range equal to shape x dtype inside the data, and the
ranges tile the data without gaps or overlaps.  Sharded checkpoints are found through
`model.safetensors.index.json` (src/safetensors.rs:347-411).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Tuple

import torch

MAX_HEADER = 100 * 1024 * 1024
MAX_SHARDS = 4096

_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1), "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    pass


class SafetensorsFile:
    """One mapped file: `entries[name] = (dtype name, shape, begin, end)`."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a safetensors header")
        self._f = open(path, "rb")
        self._map = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        (n,) = struct.unpack("<Q", self._map[:8])
        if n > MAX_HEADER or 8 + n > size:
            raise SafetensorsError(f"{path}: header length {n} does not fit the file ({size} bytes)")
        try:
            header = json.loads(self._map[8:8 + n].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"{path}: header is not JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not a JSON object")
        self.data_start = 8 + n
        data_len = size - self.data_start
        self.metadata = header.pop("__metadata__", None)
        self.entries: Dict[str, Tuple[str, Tuple[int, ...], int, int]] = {}
        spans = []
        for name, t in header.items():
            if not isinstance(t, dict) or not {"dtype", "shape", "data_offsets"} <= set(t):
                raise SafetensorsError(f"{path}: tensor {name} lacks dtype, shape or data_offsets")
            dt, shape, off = t["dtype"], t["shape"], t["data_offsets"]
            if dt not in _DTYPES:
                raise SafetensorsError(f"{path}: tensor {name} has unknown dtype {dt}")
            if (not isinstance(shape, list) or len(shape) > 4
                    or any(isinstance(d, bool) or not isinstance(d, int) or d < 0 for d in shape)):
                raise SafetensorsError(f"{path}: tensor {name} has a bad shape {shape}")
            if (not isinstance(off, list) or len(off) != 2
                    or any(isinstance(o, bool) or not isinstance(o, int) for o in off)):
                raise SafetensorsError(f"{path}: tensor {name} has bad data_offsets {off}")
            b, e = off
            count = 1
            for d in shape:
                count *= d
            if not (0 <= b <= e <= data_len):
                raise SafetensorsError(f"{path}: tensor {name} lies outside the data ({b}..{e} of {data_len})")
            if e - b != count * _DTYPES[dt][1]:
                raise SafetensorsError(
                    f"{path}: tensor {name} has {e - b} bytes, its shape {shape} of {dt} needs {count * _DTYPES[dt][1]}")
            self.entries[name] = (dt, tuple(shape), b, e)
            spans.append((b, e, name))
        spans.sort()
        at = 0
        for b, e, name in spans:
            if b != at:
                raise SafetensorsError(f"{path}: gap or overlap before tensor {name} (at byte {at}, begins {b})")
            at = e
        if at != data_len:
            raise SafetensorsError(f"{path}: {data_len - at} bytes after the last tensor")

    def names(self) -> List[str]:
        return list(self.entries)

    def shape(self, name: str) -> Tuple[int, ...]:
        return self.entries[name][1]

    def dtype(self, name: str) -> torch.dtype:
        return _DTYPES[self.entries[name][0]][0]

    def tensor(self, name: str) -> torch.Tensor:
        """A view of the mapped bytes (read-only memory: copy or move it before writing)."""
        dt, shape, b, e = self.entries[name]
        if e == b:
            return torch.empty(shape, dtype=_DTYPES[dt][0])
        buf = memoryview(self._map)[self.data_start + b:self.data_start + e]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            t = torch.frombuffer(buf, dtype=_DTYPES[dt][0])
        return t.view(shape)


class Checkpoint:
    """All tensors of a model folder, one file or shards, by name."""

    def __init__(self, model_dir: str):
        self.dir = model_dir
        index = os.path.join(model_dir, "model.safetensors.index.json")
        single = os.path.join(model_dir, "model.safetensors")
        self.files: Dict[str, SafetensorsFile] = {}
        self.where: Dict[str, str] = {}
        if os.path.exists(index):
            try:
                with open(index) as f:
                    wm = json.load(f)["weight_map"]
            except (json.JSONDecodeError, KeyError, TypeError) as e:
                raise SafetensorsError(f"{index}: no weight_map ({e})") from None
            shards = sorted(set(wm.values()))
            if len(shards) > MAX_SHARDS:
                raise SafetensorsError(f"{index}: {len(shards)} shards (at most {MAX_SHARDS})")
            for s in shards:
                if not isinstance(s, str) or os.path.basename(s) != s or s in ("", ".", ".."):
                    raise SafetensorsError(f"{index}: shard name {s!r} is not a plain file name")
                p = os.path.join(model_dir, s)
                if not os.path.exists(p):
                    raise SafetensorsError(f"{index}: shard {s} is missing")
                self.files[s] = SafetensorsFile(p)
            for s, f in self.files.items():
                for name in f.names():
                    if name in self.where:
                        raise SafetensorsError(f"tensor {name} is in two shards ({self.where[name]}, {s})")
                    self.where[name] = s
            for name, s in wm.items():
                if self.where.get(name) != s:
                    raise SafetensorsError(f"{index}: tensor {name} is not in shard {s}")
        elif os.path.exists(single):
            f = SafetensorsFile(single)
            self.files["model.safetensors"] = f
            self.where = {name: "model.safetensors" for name in f.names()}
        else:
            raise SafetensorsError(f"{model_dir} has neither model.safetensors nor model.safetensors.index.json")

    def names(self) -> List[str]:
        return list(self.where)

    def __contains__(self, name: str) -> bool:
        return name in self.where

    def shape(self, name: str):
        return self.files[self.where[name]].shape(name)

    def dtype(self, name: str):
        return self.files[self.where[name]].dtype(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self.files[self.where[name]].tensor(name)


def write_safetensors(path: str, tensors: Iterable[Tuple[str, torch.Tensor]], metadata=None) -> None:
    """Write tensors (name, CPU tensor) in the order given; data ranges tile the file."""
    tensors = list(tensors)
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    at = 0
    for name, t in tensors:
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name} has dtype {t.dtype}, which safetensors cannot hold")
        n = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [at, at + n]}
        at += n
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for _, t in tensors:
            t = t.detach().contiguous().cpu()
            f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
