"""Binding checkpoint tensors to a model by name.

A model states the tensors it needs as `TensorSpec`s (name, shape, kind).  `bind` compares
that manifest with what the checkpoint holds and raises ONE `WeightError` that lists every
missing tensor, every unexpected tensor and every wrong shape or kind, before any payload
is read.  The reference binds the same way: every name on a whitelist, asserted (rows, cols),
exact tensor count (crates/beholdd-model/src/qwen3moe.rs:807-836, :849-878).

Storage rule.  In a bfloat16 engine a floating tensor keeps bfloat16 (float16 is converted),
a tensor that the file stores in 32-bit floating point stays 32-bit, and integer tables
become int32.  In a float32 engine every floating tensor is widened to float32 (exact for
bfloat16, crates/beholdd-core/src/quant.rs:253-255).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .safetensors_io import SafetensorsReader

FLOAT_KINDS = ("F32", "BF16", "F16")
INT_KINDS = ("I32", "I64")


@dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: tuple
    init: str = "linear"      # "linear": N(0, std); "norm": 1 + N(0, std); "int": small integers
    kind: str = "float"       # "float" or "int"


class WeightError(ValueError):
    """The checkpoint does not hold exactly the tensors the model needs."""

    def __init__(self, missing, unexpected, mismatched, origin=""):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.mismatched = list(mismatched)
        lines = [f"checkpoint {origin} does not match the model:".replace("  ", " ")]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.mismatched:
            lines.append(f"  wrong shape or type ({len(self.mismatched)}):")
            lines.extend(f"    {text}" for text in self.mismatched)
        super().__init__("\n".join(lines))


def check_manifest(specs: list[TensorSpec], reader: SafetensorsReader, origin: str = "") -> None:
    wanted = {}
    for spec in specs:
        if spec.name in wanted:
            raise ValueError(f"the model names tensor {spec.name!r} twice")
        wanted[spec.name] = spec
    missing = [name for name in wanted if name not in reader.entries]
    unexpected = [name for name in reader.entries if name not in wanted]
    mismatched = []
    for name, spec in wanted.items():
        entry = reader.entries.get(name)
        if entry is None:
            continue
        if tuple(entry.shape) != tuple(spec.shape):
            mismatched.append(f"{name}: expected shape {list(spec.shape)}, checkpoint has {list(entry.shape)}")
        allowed = FLOAT_KINDS if spec.kind == "float" else INT_KINDS
        if entry.dtype not in allowed:
            mismatched.append(f"{name}: expected a {spec.kind} tensor, checkpoint has dtype {entry.dtype}")
    if missing or unexpected or mismatched:
        raise WeightError(missing, unexpected, mismatched, origin)


def stored_dtype(source_dtype: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    """The dtype a tensor is kept in on the device (see the storage rule above)."""
    if source_dtype in (torch.int32, torch.int64):
        return torch.int32
    if engine_dtype == torch.float32:
        return torch.float32
    if source_dtype == torch.float32:
        return torch.float32
    return torch.bfloat16


class BoundWeights:
    """Hands a model its tensors, one at a time, already on the device and in their kept dtype."""

    def __init__(self, reader: SafetensorsReader, engine_dtype: torch.dtype, device):
        self.reader = reader
        self.engine_dtype = engine_dtype
        self.device = device

    def planned_bytes(self, specs: list) -> int:
        """Device bytes that the tensors of `specs` will take under the storage rule, from the file's
        header alone (no payload is read)."""
        total = 0
        for spec in specs:
            entry = self.reader.entries[spec.name]
            count = 1
            for axis in entry.shape:
                count *= int(axis)
            kept = stored_dtype(entry.torch_dtype, self.engine_dtype)
            total += count * torch.empty((), dtype=kept).element_size()
        return total

    def __call__(self, name: str) -> torch.Tensor:
        source = self.reader.tensor(name)
        target = stored_dtype(source.dtype, self.engine_dtype)
        # copy=True: the result must not view the mapped file, which is closed after loading
        return source.to(device=self.device, dtype=target, copy=True).contiguous()


def bind(specs: list[TensorSpec], path: str, engine_dtype: torch.dtype, device) -> BoundWeights:
    reader = SafetensorsReader(path)
    check_manifest(specs, reader, origin=path)
    return BoundWeights(reader, engine_dtype, device)
