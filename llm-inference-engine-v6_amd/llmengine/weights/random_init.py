"""Random weights for a configuration and a seed.

Every tensor draws from a generator seeded by (seed, tensor name), so a tensor's
values do not depend on which other tensors exist or in which order they are made.
Matrices and the embedding are N(0, std); norm weights are `norm_mean` exactly
when `norm_std` is 0, else N(norm_mean, norm_std). Values are drawn in 32-bit and
then rounded to the stored dtype.

The reference has no such mode in its engine; its tests make a seeded model with
another library and save it (tests/fixtures.py:43-55).
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Any, Iterator

import torch

from ..config.registry import parse_config, resolve, architecture_name
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    return (int(seed) * 1000003 + zlib.crc32(name.encode("utf-8"))) % (2 ** 63 - 1)


def random_tensor(name: str, shape: tuple[int, ...], init: str, seed: int, dtype: torch.dtype,
                  std: float, norm_mean: float, norm_std: float) -> torch.Tensor:
    gen = torch.Generator(device="cpu")
    gen.manual_seed(_tensor_seed(seed, name))
    if init == "norm":
        if norm_std == 0.0:
            t = torch.full(shape, float(norm_mean), dtype=torch.float32)
        else:
            t = torch.randn(shape, generator=gen, dtype=torch.float32) * norm_std + norm_mean
    else:
        t = torch.randn(shape, generator=gen, dtype=torch.float32) * std
    return t.to(dtype)


def random_state(config_dict: dict, seed: int, dtype: torch.dtype = torch.bfloat16, std: float = 0.02,
                 norm_mean: float = 1.0, norm_std: float = 0.0) -> Iterator[tuple[str, torch.Tensor]]:
    """Yields (name, tensor) for every tensor the architecture's model reads."""
    arch = resolve(architecture_name(config_dict))
    model = arch.build_model(parse_config(config_dict))
    for name, spec in model.named_specs().items():
        yield name, random_tensor(name, spec.shape, spec.init, seed, dtype, std, norm_mean, norm_std)


def write_random_model(config_dict: dict, out_dir: str, seed: int, dtype: torch.dtype = torch.bfloat16,
                       std: float = 0.02, norm_mean: float = 1.0, norm_std: float = 0.0) -> str:
    """Writes a model folder (config.json, model.safetensors) and returns its path."""
    arch = resolve(architecture_name(config_dict))
    model = arch.build_model(parse_config(config_dict))
    specs = model.named_specs()
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config_dict, f, indent=2)

    def produce(name: str) -> torch.Tensor:
        s = specs[name]
        return random_tensor(name, s.shape, s.init, seed, dtype, std, norm_mean, norm_std)

    write_safetensors(os.path.join(out_dir, "model.safetensors"),
                      {n: (dtype, tuple(s.shape)) for n, s in specs.items()}, produce,
                      metadata={"format": "pt", "seed": str(seed)})
    return out_dir
