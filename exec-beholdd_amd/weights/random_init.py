"""Seeded random weights, and a model folder written from a configuration and a seed.

The reference has no random-weights mode (its tests hand-write tiny checkpoints,
crates/beholdd-model/src/qwen3moe/forward.rs:3557-3734).  Each tensor's values depend only
on (seed, tensor name), so a tensor is the same whatever else the model holds and in
whatever order tensors are drawn.  Linear and embedding weights are N(0, std); norm weights
are 1 + N(0, std).
"""

from __future__ import annotations

import hashlib
import json
import os

import numpy as np
import torch

from .binder import TensorSpec
from .safetensors_io import write_safetensors

DEFAULT_STD = 0.02


def _tensor_key(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little")


def random_tensor(spec: TensorSpec, seed: int, std: float = DEFAULT_STD) -> torch.Tensor:
    """A float32 (or int32) CPU tensor for one spec."""
    rng = np.random.Generator(np.random.Philox(key=_tensor_key(seed, spec.name)))
    if spec.kind == "int":
        return torch.from_numpy(rng.integers(0, 8, size=spec.shape, dtype=np.int32))
    values = rng.standard_normal(size=spec.shape, dtype=np.float32) * np.float32(std)
    if spec.init == "norm":
        values += np.float32(1.0)
    return torch.from_numpy(values)


def random_tensor_on_device(spec: TensorSpec, seed: int, device, dtype: torch.dtype,
                            std: float = DEFAULT_STD) -> torch.Tensor:
    """The same distributions drawn on the device, for models too large to stage through a file."""
    generator = torch.Generator(device=device)
    generator.manual_seed(_tensor_key(seed, spec.name) & 0x7FFFFFFFFFFFFFFF)
    if spec.kind == "int":
        return torch.randint(0, 8, spec.shape, device=device, dtype=torch.int32, generator=generator)
    values = torch.empty(spec.shape, device=device, dtype=dtype)
    values.normal_(0.0, std, generator=generator)
    if spec.init == "norm":
        values += 1.0
    return values


def write_random_model(folder: str, config_dict: dict, seed: int, dtype: str = "bfloat16",
                       std: float = DEFAULT_STD) -> str:
    """Write `folder/config.json` and `folder/model.safetensors` for the architecture that
    config_dict names.  `dtype` is the storage type of the floating tensors."""
    from ..registry import resolve_architecture  # late: the registry imports the models

    storage = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}.get(dtype)
    if storage is None:
        raise ValueError(f"storage dtype must be bfloat16, float32 or float16, got {dtype!r}")
    entry = resolve_architecture(config_dict)
    config = entry.config_class.from_dict(config_dict)
    model = entry.build(config)
    tensors = {}
    for spec in model.tensor_specs():
        value = random_tensor(spec, seed, std)
        tensors[spec.name] = value if spec.kind == "int" else value.to(storage)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(config_dict, handle, indent=2)
        handle.write("\n")
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder
