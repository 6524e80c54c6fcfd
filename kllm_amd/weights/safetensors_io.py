"""Reading and writing safetensors files.

Format (engine/loader/safetensors.go:1-4, :105-177): 8 bytes little-endian
header length, a JSON header ``{name: {dtype, shape, data_offsets}}`` with an
optional ``__metadata__`` entry, then the raw bytes.  The checks are the
reference's, each with its own message: header length against a cap and the
file size (:82, :117-119), unknown dtype (:44-49), negative dimension,
offsets inside the data section and in order (:160-163), byte count equal to
shape times element size (:164-167).  Sharded checkpoints are found through
``model.safetensors.index.json`` or as every ``*.safetensors`` file of the
folder; a name in two shards is an error (:240-294).

Tensors are read lazily from a memory map, so a large checkpoint is streamed
to the device one tensor at a time.
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Tuple

import torch

MAX_HEADER_BYTES = 512 << 20

_DTYPES = {
    "F64": (torch.float64, 8), "F32": (torch.float32, 4), "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2), "I64": (torch.int64, 8), "I32": (torch.int32, 4),
    "I16": (torch.int16, 2), "I8": (torch.int8, 1), "U8": (torch.uint8, 1),
    "BOOL": (torch.bool, 1),
}
_NAMES = {v[0]: k for k, v in _DTYPES.items()}


class SafetensorsError(ValueError):
    """A file that is not a well-formed safetensors file."""


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int
    end: int
    path: str

    @property
    def numel(self):
        n = 1
        for s in self.shape:
            n *= s
        return n


class SafetensorsFile:
    """One open file: its entries and a memory map of its bytes."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: too short for a header length ({size} bytes)")
        self._f = open(path, "rb")
        try:
            (hlen,) = struct.unpack("<Q", self._f.read(8))
            if hlen > MAX_HEADER_BYTES:
                raise SafetensorsError(f"{path}: header length {hlen} exceeds {MAX_HEADER_BYTES}")
            if hlen > size - 8:
                raise SafetensorsError(
                    f"{path}: header length {hlen} is larger than the file ({size} bytes)")
            try:
                header = json.loads(self._f.read(hlen).decode("utf-8"))
            except (UnicodeDecodeError, json.JSONDecodeError) as e:
                raise SafetensorsError(f"{path}: header is not valid JSON ({e})") from None
            if not isinstance(header, dict):
                raise SafetensorsError(f"{path}: header is not a JSON object")
            self.data_start = 8 + hlen
            data_len = size - self.data_start
            self.metadata = header.pop("__metadata__", None) or {}
            self.entries: Dict[str, TensorEntry] = {}
            for name, info in header.items():
                self.entries[name] = self._entry(name, info, data_len)
            self._mm = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ) if size else None
        except Exception:
            self._f.close()
            raise

    def _entry(self, name, info, data_len) -> TensorEntry:
        path = self.path
        if not isinstance(info, dict) or not {"dtype", "shape", "data_offsets"} <= set(info):
            raise SafetensorsError(f"{path}: entry {name!r} lacks dtype, shape or data_offsets")
        dtype = info["dtype"]
        if dtype not in _DTYPES:
            raise SafetensorsError(f"{path}: tensor {name!r} has unknown dtype {dtype!r}")
        shape = info["shape"]
        if not isinstance(shape, list) or any(
                isinstance(s, bool) or not isinstance(s, int) for s in shape):
            raise SafetensorsError(f"{path}: tensor {name!r} has a malformed shape {shape!r}")
        if any(s < 0 for s in shape):
            raise SafetensorsError(f"{path}: tensor {name!r} has a negative dimension {shape}")
        offs = info["data_offsets"]
        if (not isinstance(offs, list) or len(offs) != 2
                or any(isinstance(o, bool) or not isinstance(o, int) for o in offs)):
            raise SafetensorsError(f"{path}: tensor {name!r} has malformed data_offsets {offs!r}")
        begin, end = offs
        if begin < 0 or end < begin or end > data_len:
            raise SafetensorsError(
                f"{path}: tensor {name!r} offsets [{begin}, {end}) lie outside the data "
                f"section of {data_len} bytes")
        numel = 1
        for s in shape:
            numel *= s
        want = numel * _DTYPES[dtype][1]
        if end - begin != want:
            raise SafetensorsError(
                f"{path}: tensor {name!r} has {end - begin} bytes, its shape {shape} and dtype "
                f"{dtype} need {want}")
        return TensorEntry(name, dtype, tuple(shape), begin, end, path)

    def read(self, name: str) -> torch.Tensor:
        """The tensor as a CPU tensor backed by the memory map (read-only:
        copy or move it before writing to it)."""
        e = self.entries[name]
        tdtype = _DTYPES[e.dtype][0]
        if e.numel == 0:
            return torch.empty(e.shape, dtype=tdtype)
        buf = memoryview(self._mm)[self.data_start + e.begin:self.data_start + e.end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the buffer is not writable
            flat = torch.frombuffer(buf, dtype=tdtype, count=e.numel)
        return flat.reshape(e.shape)

    def close(self):
        # Tensors handed out by read() keep the map alive through the buffer
        # protocol; closing then only drops this object's own references.
        try:
            if self._mm is not None:
                self._mm.close()
        except BufferError:
            pass
        self._mm = None
        self._f.close()


class Checkpoint:
    """Every tensor of a model folder (or of one file), whichever shard holds it."""

    def __init__(self, path: str):
        self.files: List[SafetensorsFile] = []
        self.entries: Dict[str, TensorEntry] = {}
        self._by_path: Dict[str, SafetensorsFile] = {}
        for p in self._shard_paths(path):
            f = SafetensorsFile(p)
            self.files.append(f)
            self._by_path[p] = f
            for name, e in f.entries.items():
                if name in self.entries:
                    self.close()
                    raise SafetensorsError(
                        f"tensor {name!r} appears in both {self.entries[name].path} and {p}")
                self.entries[name] = e

    @staticmethod
    def _shard_paths(path: str) -> List[str]:
        if os.path.isfile(path):
            return [path]
        if not os.path.isdir(path):
            raise SafetensorsError(f"{path}: no such file or folder")
        index = os.path.join(path, "model.safetensors.index.json")
        if os.path.isfile(index):
            try:
                with open(index, "r", encoding="utf-8") as f:
                    wm = json.load(f)["weight_map"]
                names = sorted(set(wm.values()))
            except (KeyError, AttributeError, TypeError, json.JSONDecodeError) as e:
                raise SafetensorsError(f"{index}: malformed index ({e})") from None
            paths = [os.path.join(path, n) for n in names]
        else:
            paths = sorted(os.path.join(path, n) for n in os.listdir(path)
                           if n.endswith(".safetensors"))
        if not paths:
            raise SafetensorsError(f"{path}: no .safetensors file found")
        for p in paths:
            if not os.path.isfile(p):
                raise SafetensorsError(f"{p}: shard named by the index is missing")
        return paths

    def names(self):
        return sorted(self.entries)

    def read(self, name: str) -> torch.Tensor:
        return self._by_path[self.entries[name].path].read(name)

    def close(self):
        for f in self.files:
            f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata=None):
    """Write ``tensors`` (CPU or device tensors) in the order given."""
    header = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    for name, t in tensors.items():
        if t.dtype not in _NAMES:
            raise SafetensorsError(f"tensor {name!r}: dtype {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t in tensors.items():
            c = t.detach().to("cpu").contiguous()
            if c.numel():
                f.write(c.reshape(-1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
