"""Random weights from a configuration and a seed.

Matrices are N(0, std) (std 0.02 unless given), norm weights are 1. Every
tensor has a generator of its own, seeded by (seed, position of the tensor in
the model's list), so a tensor's values do not depend on the others' sizes.
The reference has random weights only as a test fixture
(tests/common/mod.rs:632-731).
"""
from __future__ import annotations

import os
from typing import Dict, Iterator, Tuple

import torch

from ..config import save_config
from ..parts.base import WeightSpec
from .safetensors_io import LazyTensor, write_safetensors


def _make(spec: WeightSpec, seed: int, index: int, std: float, dtype: torch.dtype, device) -> torch.Tensor:
    if spec.kind == "table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "ones":
        return torch.ones(spec.shape, dtype=dtype, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    if spec.init != "normal":
        raise ValueError(f"unknown init '{spec.init}'")
    generator = torch.Generator(device=device)
    generator.manual_seed((int(seed) * 1_000_003 + index) & 0x7FFF_FFFF_FFFF_FFFF)
    values = torch.empty(spec.shape, dtype=torch.float32, device=device)
    values.normal_(0.0, std, generator=generator)
    return values.to(dtype)


def random_tensors(specs: Dict[str, WeightSpec], seed: int, std: float = 0.02,
                   dtype: torch.dtype = torch.bfloat16, device="cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    """(name, tensor) for every spec, in the order of `specs`, made on `device`."""
    for index, (name, spec) in enumerate(specs.items()):
        yield name, _make(spec, seed, index, std, dtype, device)


def write_random_model(config, folder: str, seed: int, std: float = 0.02,
                       dtype: torch.dtype = torch.bfloat16) -> str:
    """Write `folder/config.json` and `folder/model.safetensors` for `config`."""
    from ..config import architecture

    spec = architecture(config.architecture).build(config)
    specs = spec.weight_specs()
    lazy = {}
    for index, (name, weight) in enumerate(specs.items()):
        stored = torch.int32 if weight.kind == "table" else dtype
        lazy[name] = LazyTensor(
            stored, weight.shape,
            lambda weight=weight, index=index: _make(weight, seed, index, std, dtype, "cpu"))
    os.makedirs(folder, exist_ok=True)
    save_config(config, folder)
    write_safetensors(os.path.join(folder, "model.safetensors"), lazy,
                      metadata={"format": "pt", "seed": seed})
    return folder
