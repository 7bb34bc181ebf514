"""Reader and writer of the safetensors file format.

File = 8-byte little-endian header length, a JSON header
{name: {dtype, shape, data_offsets: [begin, end]}}, then the raw little-endian
tensor bytes. The reader checks the file the way the reference's GGUF parser
checks its own (crates/xrt-gguf/src/lib.rs:268-290, 331-415: magic/length,
duplicate names, zero dimensions, data past the end of the file) and looks
tensors up by exact name (crates/xrt-gguf/src/lib.rs:532-541).
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, Tuple

import numpy as np
import torch


class SafetensorsError(ValueError):
    """A file that is not a well-formed safetensors file."""


# dtype name in the file -> (bytes per element, numpy dtype used to view the bytes)
_DTYPES = {
    "F32": (4, np.float32),
    "F16": (2, np.float16),
    "BF16": (2, np.uint16),     # numpy has no bfloat16: viewed as bits
    "I32": (4, np.int32),
    "I64": (8, np.int64),
}

_TORCH_TO_NAME = {
    torch.float32: "F32",
    torch.float16: "F16",
    torch.bfloat16: "BF16",
    torch.int32: "I32",
    torch.int64: "I64",
}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int      # byte offsets relative to the start of the data section
    end: int


class SafetensorsFile:
    """A memory-mapped safetensors file with its parsed, validated header."""

    def __init__(self, path: str):
        self.path = path
        if not os.path.isfile(path):
            raise SafetensorsError(f"{path}: no such file")
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"{path}: truncated (no header length)")
        self._handle = open(path, "rb")
        self._map = mmap.mmap(self._handle.fileno(), 0, access=mmap.ACCESS_READ)
        (header_len,) = struct.unpack("<Q", self._map[:8])
        if header_len > size - 8:
            raise SafetensorsError(
                f"{path}: header length {header_len} exceeds the file size {size}")
        try:
            header = json.loads(self._map[8:8 + header_len].decode("utf-8"),
                                object_pairs_hook=_reject_duplicates)
        except (UnicodeDecodeError, json.JSONDecodeError) as error:
            raise SafetensorsError(f"{path}: invalid header JSON: {error}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{path}: header is not a JSON object")
        self.metadata = header.pop("__metadata__", None) or {}
        self._data_start = 8 + header_len
        data_size = size - self._data_start
        self.entries: Dict[str, TensorEntry] = {}
        for name, info in header.items():
            self.entries[name] = _parse_entry(path, name, info, data_size)
        _check_overlap(path, self.entries.values())

    def names(self):
        return list(self.entries)

    def __contains__(self, name: str) -> bool:
        return name in self.entries

    def entry(self, name: str) -> TensorEntry:
        if name not in self.entries:
            raise SafetensorsError(f"{self.path}: missing tensor {name}")
        return self.entries[name]

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor with a copy of the tensor's bytes, in the stored dtype."""
        entry = self.entry(name)
        _, np_dtype = _DTYPES[entry.dtype]
        start = self._data_start + entry.begin
        count = int(np.prod(entry.shape, dtype=np.int64)) if entry.shape else 1
        array = np.frombuffer(self._map, dtype=np_dtype, count=count, offset=start).copy()
        tensor = torch.from_numpy(array)
        if entry.dtype == "BF16":
            tensor = tensor.view(torch.bfloat16)
        return tensor.reshape(entry.shape)

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._handle.close()
            self._map = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def _reject_duplicates(pairs):
    seen = {}
    for key, value in pairs:
        if key in seen:
            raise SafetensorsError(f"duplicate tensor name {key}")
        seen[key] = value
    return seen


def _parse_entry(path: str, name: str, info, data_size: int) -> TensorEntry:
    if not isinstance(info, dict) or not {"dtype", "shape", "data_offsets"} <= set(info):
        raise SafetensorsError(f"{path}: tensor {name}: header entry lacks dtype/shape/data_offsets")
    dtype = info["dtype"]
    if dtype not in _DTYPES:
        raise SafetensorsError(f"{path}: tensor {name}: unsupported dtype {dtype}")
    shape = info["shape"]
    if not isinstance(shape, list) or any(
            isinstance(d, bool) or not isinstance(d, int) or d < 0 for d in shape):
        raise SafetensorsError(f"{path}: tensor {name}: invalid shape {shape!r}")
    offsets = info["data_offsets"]
    if (not isinstance(offsets, list) or len(offsets) != 2
            or any(isinstance(o, bool) or not isinstance(o, int) for o in offsets)):
        raise SafetensorsError(f"{path}: tensor {name}: invalid data_offsets {offsets!r}")
    begin, end = offsets
    if begin < 0 or end < begin or end > data_size:
        raise SafetensorsError(
            f"{path}: tensor {name}: bytes [{begin}, {end}) lie outside the data section of {data_size} bytes")
    count = 1
    for d in shape:
        count *= d
    if count * _DTYPES[dtype][0] != end - begin:
        raise SafetensorsError(
            f"{path}: tensor {name}: shape {shape} of {dtype} needs {count * _DTYPES[dtype][0]} bytes, "
            f"the header gives {end - begin}")
    return TensorEntry(name, dtype, tuple(shape), begin, end)


def _check_overlap(path: str, entries: Iterable[TensorEntry]) -> None:
    ordered = sorted((e for e in entries if e.end > e.begin), key=lambda e: e.begin)
    for before, after in zip(ordered, ordered[1:]):
        if after.begin < before.end:
            raise SafetensorsError(
                f"{path}: tensors {before.name} and {after.name} overlap in the data section")


def write_safetensors(path: str, tensors, metadata=None) -> None:
    """Write (name, tensor) pairs, in the given order, as one safetensors file.

    `tensors` may be a dict or any iterable of pairs; each tensor is moved to
    the CPU and written when its turn comes, so a generator keeps memory flat.
    A first pass over a dict fixes the header; a generator must therefore come
    with its layout: pass a dict of lazily produced tensors via `LazyTensors`.
    """
    items = tensors.items() if isinstance(tensors, dict) else list(tensors)
    header = {}
    offset = 0
    layout = []
    for name, tensor in items:
        spec = tensor if isinstance(tensor, LazyTensor) else None
        dtype = spec.dtype if spec else tensor.dtype
        shape = tuple(spec.shape if spec else tensor.shape)
        if dtype not in _TORCH_TO_NAME:
            raise SafetensorsError(f"tensor {name}: dtype {dtype} cannot be written")
        if name in header:
            raise SafetensorsError(f"duplicate tensor name {name}")
        count = 1
        for d in shape:
            count *= d
        nbytes = count * _DTYPES[_TORCH_TO_NAME[dtype]][0]
        header[name] = {"dtype": _TORCH_TO_NAME[dtype], "shape": list(shape),
                        "data_offsets": [offset, offset + nbytes]}
        layout.append((name, tensor, nbytes))
        offset += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)))
        handle.write(blob)
        for name, tensor, nbytes in layout:
            if isinstance(tensor, LazyTensor):
                tensor = tensor.make()
            data = tensor.detach().to("cpu").contiguous()
            if data.dtype == torch.bfloat16:
                data = data.view(torch.int16)
            raw = data.numpy().tobytes()
            if len(raw) != nbytes:
                raise SafetensorsError(f"tensor {name}: produced {len(raw)} bytes, expected {nbytes}")
            handle.write(raw)


class LazyTensor:
    """A tensor of known dtype and shape that is produced only when it is written."""

    def __init__(self, dtype: torch.dtype, shape, make):
        self.dtype = dtype
        self.shape = tuple(shape)
        self.make = make
