"""Random weights from a configuration and a seed.

Matrices are N(0, std) (std 0.02 unless given), norm weights are 1 (or 1 + N(0, gain_std)).
Every element comes from a counter-based generator keyed by (seed, tensor name, element
index): a tensor's values depend neither on the other tensors nor on where or in what
pieces they are made, so the folder that `write_random_model` writes, the weights that
`Engine.random` makes on the GPU and the ones `make_tensor` makes on the host are the same
bit for bit.

The generator: key = mix(mix(seed) ^ sha256(name)[:8]); element i draws the two 64-bit words
mix(key + 2i*G) and mix(key + (2i+1)*G) (mix: the splitmix64 step, G its increment), adds up
twelve 10-bit fields of them (six a word) and centres the sum: twelve uniform numbers make a
normal one to within a few per cent of density out to six deviations, and integers add up
the same way everywhere. value = float32(2*sum - 12*1023) * float32(std / (2*sqrt(1024^2 - 1))),
rounded to the stored type to nearest even. The kernel `xrt_random_normal` does the same on
the GPU.

The reference has random weights only as a test fixture (tests/common/mod.rs:632-731).
"""
from __future__ import annotations

import hashlib
import math
import os
from typing import Dict, Iterator, Tuple

import torch

from ..config import save_config
from ..parts.base import WeightSpec
from .safetensors_io import LazyTensor, write_safetensors

_MASK = (1 << 64) - 1
_GOLDEN = 0x9E3779B97F4A7C15
_CHUNK = 1 << 18            # elements made at a time on the host: what stays in the processor's caches


def _mix(value: int) -> int:
    """One splitmix64 step on a Python integer."""
    value = (value + _GOLDEN) & _MASK
    value = ((value ^ (value >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    value = ((value ^ (value >> 27)) * 0x94D049BB133111EB) & _MASK
    return value ^ (value >> 31)


def tensor_key(seed: int, name: str) -> int:
    """The 64-bit key of one tensor's stream."""
    name_word = int.from_bytes(hashlib.sha256(name.encode("utf-8")).digest()[:8], "little")
    return _mix(_mix(int(seed) & _MASK) ^ name_word)


def normal_scale(std: float) -> float:
    """What the centred sum of twelve 10-bit fields is multiplied by to have deviation `std` (as float32)."""
    return float(torch.tensor(std / (2.0 * math.sqrt(1024.0 * 1024.0 - 1.0)), dtype=torch.float32))


def _signed(value: int) -> int:
    """A 64-bit pattern as the signed integer that torch's int64 holds for it."""
    value &= _MASK
    return value - (1 << 64) if value >= (1 << 63) else value


# 64-bit arithmetic on int64 tensors: sums and products wrap, and a shift to the right is made logical by
# masking off the sign bits it drags in.
_G, _C1, _C2 = _signed(_GOLDEN), _signed(0xBF58476D1CE4E5B9), _signed(0x94D049BB133111EB)
_FIELDS_0_2_4 = 1023 | (1023 << 20) | (1023 << 40)


def _mix_tensor(words: torch.Tensor) -> torch.Tensor:
    """One splitmix64 step on every element, in place."""
    words.add_(_G)
    words.bitwise_xor_((words >> 30).bitwise_and_((1 << 34) - 1)).mul_(_C1)
    words.bitwise_xor_((words >> 27).bitwise_and_((1 << 37) - 1)).mul_(_C2)
    return words.bitwise_xor_((words >> 31).bitwise_and_((1 << 33) - 1))


def _field_sum(words: torch.Tensor) -> torch.Tensor:
    """The sum of the six lowest 10-bit fields of every element: fields 0, 2, 4 and 1, 3, 5 are added in
    lanes of twenty bits, then the three lanes."""
    lanes = (words & _FIELDS_0_2_4).add_((words >> 10).bitwise_and_(_FIELDS_0_2_4))
    return lanes.add_(lanes >> 20).add_(lanes >> 40).bitwise_and_((1 << 20) - 1)


def normal_values(key: int, first: int, count: int, scale: float) -> torch.Tensor:
    """float32 values of elements first .. first + count of the stream `key` (scale as float32)."""
    base = torch.arange(first, first + count, dtype=torch.int64).mul_(_signed(2 * _GOLDEN)).add_(_signed(key))
    second = base + _G
    total = _field_sum(_mix_tensor(base)).add_(_field_sum(_mix_tensor(second)))
    return total.mul_(2).sub_(12 * 1023).to(torch.float32).mul_(scale)


def make_tensor(spec: WeightSpec, seed: int, name: str, std: float, dtype: torch.dtype,
                gain_std: float = 0.0) -> torch.Tensor:
    """The tensor `name` on the host, in `dtype` (integer tables: zeros, int32)."""
    if spec.kind == "table":
        return torch.zeros(spec.shape, dtype=torch.int32)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype)
    if spec.init == "ones" and gain_std == 0.0:
        return torch.ones(spec.shape, dtype=dtype)
    if spec.init not in ("normal", "ones"):
        raise ValueError(f"unknown init '{spec.init}'")
    count = math.prod(spec.shape)
    key = tensor_key(seed, name)
    scale = normal_scale(gain_std if spec.init == "ones" else std)
    out = torch.empty(count, dtype=dtype)
    for first in range(0, count, _CHUNK):
        piece = normal_values(key, first, min(_CHUNK, count - first), scale)
        if spec.init == "ones":
            piece = piece + 1.0
        out[first:first + piece.numel()] = piece.to(dtype)
    return out.reshape(spec.shape)


def make_tensor_on_device(ops, spec: WeightSpec, seed: int, name: str, std: float, dtype: torch.dtype, device,
                          gain_std: float = 0.0) -> torch.Tensor:
    """The same tensor made where it is needed: by the kernel library on a GPU, on the host otherwise."""
    device = torch.device(device)
    plain = spec.kind == "table" or spec.init == "zeros" or (spec.init == "ones" and gain_std == 0.0)
    if device.type != "cuda" or plain or not hasattr(ops, "random_normal"):
        return make_tensor(spec, seed, name, std, dtype, gain_std).to(device)
    if spec.init not in ("normal", "ones"):
        raise ValueError(f"unknown init '{spec.init}'")
    out = torch.empty(spec.shape, dtype=dtype, device=device)
    is_gain = spec.init == "ones"
    ops.random_normal(out, tensor_key(seed, name), normal_scale(gain_std if is_gain else std), 1.0 if is_gain else 0.0)
    return out


class RandomSource:
    """Random tensors by name, each made when a part asks for it: on the GPU by the kernel library where
    the model lives there, else on the host; `host(name)` makes the same tensor on the host."""

    def __init__(self, specs: Dict[str, WeightSpec], seed: int, std: float, dtype: torch.dtype, device, ops=None,
                 gain_std: float = 0.0):
        self.specs = dict(specs)
        self.seed, self.std, self.dtype, self.gain_std = int(seed), float(std), dtype, float(gain_std)
        self.device = torch.device(device)
        self.ops = ops

    def __contains__(self, name: str) -> bool:
        return name in self.specs

    def keys(self):
        return self.specs.keys()

    def __getitem__(self, name: str) -> torch.Tensor:
        if name not in self.specs:
            raise KeyError(name)
        return make_tensor_on_device(self.ops, self.specs[name], self.seed, name, self.std, self.dtype, self.device,
                                     self.gain_std)

    def host(self, name: str) -> torch.Tensor:
        if name not in self.specs:
            raise KeyError(name)
        return make_tensor(self.specs[name], self.seed, name, self.std, self.dtype, self.gain_std)


def random_tensors(specs: Dict[str, WeightSpec], seed: int, std: float = 0.02,
                   dtype: torch.dtype = torch.bfloat16, gain_std: float = 0.0) -> Iterator[Tuple[str, torch.Tensor]]:
    """(name, tensor) for every spec, in the order of `specs`, made on the host."""
    for name, spec in specs.items():
        yield name, make_tensor(spec, seed, name, std, dtype, gain_std)


def write_random_model(config, folder: str, seed: int, std: float = 0.02,
                       dtype: torch.dtype = torch.bfloat16, gain_std: float = 0.0) -> str:
    """Write `folder/config.json` and `folder/model.safetensors` for `config`."""
    from ..config import architecture

    spec = architecture(config.architecture).build(config)
    specs = spec.weight_specs()
    lazy = {}
    for name, weight in specs.items():
        stored = torch.int32 if weight.kind == "table" else dtype
        lazy[name] = LazyTensor(
            stored, weight.shape,
            lambda weight=weight, name=name: make_tensor(weight, seed, name, std, dtype, gain_std))
    os.makedirs(folder, exist_ok=True)
    save_config(config, folder)
    write_safetensors(os.path.join(folder, "model.safetensors"), lazy,
                      metadata={"format": "pt", "seed": seed})
    return folder
