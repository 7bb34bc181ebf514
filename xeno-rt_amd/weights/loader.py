"""Bind the tensors of a model folder to a model, by name.

The reference resolves every tensor by exact name at load and fails on the
first that is missing (crates/xrt-models/src/llama.rs:286-337,
crates/xrt-gguf/src/lib.rs:532-541). Here the whole set is compared at once:
one error lists the missing tensors, the unexpected ones and the wrong shapes.

Kept precision: tensors are handed on as the file stores them (BF16, F16, F32;
64-bit integer tables become int32). Conversion to the compute dtype is the
business of the part that binds the tensor, so that the 32-bit path widens an
F16 checkpoint exactly and only the bfloat16 path rounds it.

`CheckpointSource` hands out one tensor at a time, read from the mapped file
when a part asks for it and kept by nobody: a model's weights are on the device
once, in the form the parts bound them, and `Engine.get_tensor` reads the file
again.
"""
from __future__ import annotations

import json
import os
import warnings
from typing import Dict, Iterable, List, Optional

import torch

from ..parts.base import WeightSpec
from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightError(ValueError):
    """The tensors of a checkpoint do not fit the model."""

    def __init__(self, where: str, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.wrong_dtype = sorted(wrong_dtype)
        lines = [f"{where}: the checkpoint does not fit the model"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{name} expected {list(want)} found {list(found)}" for name, want, found in self.wrong_shape))
        if self.wrong_dtype:
            lines.append(f"  wrong dtypes ({len(self.wrong_dtype)}): " + "; ".join(
                f"{name} is {found}, a {kind} needs {need}" for name, kind, found, need in self.wrong_dtype))
        super().__init__("\n".join(lines))


_FLOAT = ("F32", "F16", "BF16")
_INTEGER = ("I32", "I64")


def _kept(tensor: torch.Tensor) -> torch.Tensor:
    if tensor.dtype == torch.int64:
        if tensor.numel() and (int(tensor.max()) > 2**31 - 1 or int(tensor.min()) < -2**31):
            raise SafetensorsError("integer table does not fit int32")
        return tensor.to(torch.int32)
    return tensor


class CheckpointFiles:
    """The safetensors files of a folder: model.safetensors, or the shards that
    model.safetensors.index.json names."""

    def __init__(self, folder: str):
        self.folder = folder
        index_path = os.path.join(folder, "model.safetensors.index.json")
        single = os.path.join(folder, "model.safetensors")
        self.files: List[SafetensorsFile] = []
        self.where: Dict[str, SafetensorsFile] = {}
        if os.path.isfile(index_path):
            with open(index_path) as handle:
                weight_map = json.load(handle).get("weight_map", {})
            opened: Dict[str, SafetensorsFile] = {}
            for name, shard in weight_map.items():
                if shard not in opened:
                    opened[shard] = SafetensorsFile(os.path.join(folder, shard))
                    self.files.append(opened[shard])
            for file in self.files:
                for name in file.names():
                    if name in self.where:
                        raise SafetensorsError(f"{folder}: tensor {name} is in two shards")
                    self.where[name] = file
        elif os.path.isfile(single):
            file = SafetensorsFile(single)
            self.files.append(file)
            self.where = {name: file for name in file.names()}
        else:
            raise SafetensorsError(f"{folder}: no model.safetensors and no model.safetensors.index.json")

    def close(self):
        for file in self.files:
            file.close()


def check_names(where: str, expected: Dict[str, WeightSpec], found: Dict[str, tuple],
                ignored: Iterable[str] = ()) -> None:
    """Raise one WeightError if `found` (name -> (dtype name, shape)) does not fit `expected`."""
    ignored = set(ignored)
    missing = [name for name in expected if name not in found]
    unexpected = [name for name in found if name not in expected and name not in ignored]
    wrong_shape, wrong_dtype = [], []
    for name, spec in expected.items():
        if name not in found:
            continue
        dtype, shape = found[name]
        if tuple(shape) != tuple(spec.shape):
            wrong_shape.append((name, tuple(spec.shape), tuple(shape)))
        if spec.kind == "table" and dtype not in _INTEGER:
            wrong_dtype.append((name, spec.kind, dtype, "/".join(_INTEGER)))
        if spec.kind != "table" and dtype not in _FLOAT:
            wrong_dtype.append((name, spec.kind, dtype, "/".join(_FLOAT)))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(where, missing, unexpected, wrong_shape, wrong_dtype)


def warn_of_ignored(where: str, found: Iterable[str], ignored: Iterable[str]) -> None:
    """A checkpoint may carry tensors that the model says it does not read (the head's matrix of a model
    that ties it to the embedding, llama.rs:301-305): they are left alone, and said so once."""
    present = sorted(set(ignored) & set(found))
    if present:
        warnings.warn(f"{where}: {', '.join(present)} ignored: the model does not read "
                      f"{'it' if len(present) == 1 else 'them'} (a tied head uses the embedding's table)", stacklevel=3)


class CheckpointSource:
    """The tensors of a model folder by name, each read when it is asked for (on the host, as stored).

    The whole set of names, shapes and dtypes is checked against `expected` when the source is made.
    The files stay open (mapped) until `release()`: whoever has bound what it needs calls it; a tensor
    asked for after that opens its file again for the one read."""

    def __init__(self, folder: str, expected: Dict[str, WeightSpec], ignored: Iterable[str] = ()):
        self.folder = folder
        self.expected = dict(expected)
        self.files: Optional[CheckpointFiles] = CheckpointFiles(folder)
        try:
            found = {name: (file.entries[name].dtype, file.entries[name].shape)
                     for name, file in self.files.where.items()}
            check_names(folder, self.expected, found, ignored)
            warn_of_ignored(folder, found, ignored)
        except Exception:
            self.files.close()
            raise

    def __contains__(self, name: str) -> bool:
        return name in self.expected

    def keys(self):
        return self.expected.keys()

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self.expected:
            raise KeyError(name)
        if self.files is not None:
            return _kept(self.files.where[name].read(name))
        files = CheckpointFiles(self.folder)            # released: open, read the one tensor, close
        try:
            return _kept(files.where[name].read(name))
        finally:
            files.close()

    def host(self, name: str) -> torch.Tensor:
        return self[name]

    @property
    def is_open(self) -> bool:
        return self.files is not None

    def release(self) -> None:
        """Close the files; tensors can still be asked for, one file opening each."""
        if self.files is not None:
            self.files.close()
            self.files = None

    close = release


def load_tensors(folder: str, expected: Dict[str, WeightSpec], ignored: Iterable[str] = (),
                 device="cpu") -> Dict[str, torch.Tensor]:
    """All expected tensors of `folder` on `device`, after the whole set has been checked."""
    files = CheckpointFiles(folder)
    try:
        found = {name: (file.entries[name].dtype, file.entries[name].shape)
                 for name, file in files.where.items()}
        check_names(folder, expected, found, ignored)
        warn_of_ignored(folder, found, ignored)
        tensors = {}
        for name in expected:
            tensors[name] = _kept(files.where[name].read(name)).to(device)
        return tensors
    finally:
        files.close()
