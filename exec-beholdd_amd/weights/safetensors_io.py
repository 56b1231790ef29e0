"""A checked safetensors reader and a writer.

The file format: an 8-byte little-endian header length, a JSON object that maps each tensor
name to {dtype, shape, data_offsets}, then the tensors' bytes.  The checks are the ones the
reference's reader makes (crates/beholdd-format/src/safetensors.rs:96-169 open, :258-296 layout,
:333-421 header and entries): a header of 0 or more than 512 MiB is refused, an unknown dtype
is refused (not skipped), byte length must equal dtype size times element count, tensors may
not overlap, leave holes or trailing bytes, and a name may not occur in two shards.
Tensors are memory-mapped and copied only when a caller asks for them.
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass

import torch

MAX_HEADER_BYTES = 512 * 1024 * 1024

# safetensors dtype string -> (torch dtype, bytes per element)
DTYPES = {
    "F32": (torch.float32, 4),
    "BF16": (torch.bfloat16, 2),
    "F16": (torch.float16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
_NAMES = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16",
          torch.int32: "I32", torch.int64: "I64"}


class SafetensorsError(ValueError):
    """The file is not a well-formed safetensors checkpoint."""


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str            # the safetensors dtype string
    shape: tuple
    shard: int            # index into the reader's shard list
    begin: int            # byte offsets inside the shard file
    end: int

    @property
    def torch_dtype(self):
        return DTYPES[self.dtype][0]


class SafetensorsReader:
    """All tensors of one file, or of every `*.safetensors` file of a folder in sorted order."""

    def __init__(self, path: str):
        if os.path.isdir(path):
            files = sorted(os.path.join(path, f) for f in os.listdir(path) if f.endswith(".safetensors"))
            if not files:
                raise SafetensorsError(f"{path}: the folder holds no .safetensors file")
        else:
            files = [path]
        self.files = files
        self.entries: dict[str, TensorEntry] = {}
        self._maps: list = [None] * len(files)
        self._handles: list = [None] * len(files)
        for shard, file in enumerate(files):
            for entry in self._read_shard(file, shard):
                if entry.name in self.entries:
                    other = files[self.entries[entry.name].shard]
                    raise SafetensorsError(f"tensor {entry.name!r} occurs in both {other} and {file}")
                self.entries[entry.name] = entry

    # ---- header ----
    @staticmethod
    def _read_shard(file: str, shard: int) -> list[TensorEntry]:
        try:
            size = os.path.getsize(file)
            with open(file, "rb") as handle:
                prefix = handle.read(8)
                if len(prefix) != 8:
                    raise SafetensorsError(f"{file}: shorter than the 8-byte header length")
                (header_len,) = struct.unpack("<Q", prefix)
                if header_len == 0 or header_len > MAX_HEADER_BYTES:
                    raise SafetensorsError(f"{file}: header length {header_len} is outside 1..{MAX_HEADER_BYTES}")
                if 8 + header_len > size:
                    raise SafetensorsError(f"{file}: header of {header_len} bytes runs past the end of the file")
                raw = handle.read(header_len)
        except FileNotFoundError:
            raise SafetensorsError(f"{file}: no such file") from None
        try:
            header = json.loads(raw.decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as error:
            raise SafetensorsError(f"{file}: header is not valid JSON ({error})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"{file}: header must be a JSON object")
        data_start = 8 + header_len
        data_len = size - data_start
        entries = []
        for name, meta in header.items():
            if name == "__metadata__":
                continue
            entries.append(SafetensorsReader._parse_entry(file, shard, name, meta, data_start, data_len))
        # layout: no overlap, no hole, no trailing bytes
        cursor = data_start
        for entry in sorted(entries, key=lambda e: (e.begin, e.end)):
            if entry.begin < cursor:
                raise SafetensorsError(f"{file}: tensor {entry.name!r} overlaps the tensor before it")
            if entry.begin > cursor:
                raise SafetensorsError(f"{file}: {entry.begin - cursor} unused bytes before tensor {entry.name!r}")
            cursor = entry.end
        if cursor != size:
            raise SafetensorsError(f"{file}: {size - cursor} trailing bytes after the last tensor")
        return entries

    @staticmethod
    def _parse_entry(file, shard, name, meta, data_start, data_len) -> TensorEntry:
        if not isinstance(meta, dict):
            raise SafetensorsError(f"{file}: entry {name!r} must be an object")
        dtype = meta.get("dtype")
        if dtype not in DTYPES:
            raise SafetensorsError(f"{file}: tensor {name!r} has dtype {dtype!r}; supported: {sorted(DTYPES)}")
        shape = meta.get("shape")
        if not isinstance(shape, list) or any(isinstance(a, bool) or not isinstance(a, int) or a < 0 for a in shape):
            raise SafetensorsError(f"{file}: tensor {name!r} has a malformed shape {shape!r}")
        offsets = meta.get("data_offsets")
        if (not isinstance(offsets, list) or len(offsets) != 2
                or any(isinstance(o, bool) or not isinstance(o, int) or o < 0 for o in offsets)):
            raise SafetensorsError(f"{file}: tensor {name!r} has malformed data_offsets {offsets!r}")
        begin, end = offsets
        if end < begin:
            raise SafetensorsError(f"{file}: tensor {name!r} has reversed data_offsets {offsets!r}")
        if end > data_len:
            raise SafetensorsError(f"{file}: tensor {name!r} ends at byte {end} of a {data_len}-byte data section")
        count = 1
        for axis in shape:
            count *= axis
        expected = count * DTYPES[dtype][1]
        if end - begin != expected:
            raise SafetensorsError(
                f"{file}: tensor {name!r} of dtype {dtype} and shape {shape} needs {expected} bytes, "
                f"the file gives {end - begin}")
        return TensorEntry(name, dtype, tuple(shape), shard, data_start + begin, data_start + end)

    # ---- data ----
    def names(self) -> list[str]:
        return list(self.entries)

    def _map(self, shard: int):
        if self._maps[shard] is None:
            handle = open(self.files[shard], "rb")
            self._handles[shard] = handle
            # a private copy-on-write mapping: torch wants a writable buffer, the file is never changed
            self._maps[shard] = mmap.mmap(handle.fileno(), 0, access=mmap.ACCESS_COPY)
        return self._maps[shard]

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor that views the mapped file (no copy); keep the reader alive while it is used."""
        entry = self.entries[name]
        torch_dtype, width = DTYPES[entry.dtype]
        count = (entry.end - entry.begin) // width
        if count == 0:
            return torch.empty(entry.shape, dtype=torch_dtype)
        flat = torch.frombuffer(self._map(entry.shard), dtype=torch_dtype, count=count, offset=entry.begin)
        return flat.reshape(entry.shape)

    def close(self):
        for index, mapped in enumerate(self._maps):
            if mapped is not None:
                try:
                    mapped.close()
                except BufferError:
                    pass  # a tensor still views it; the mapping goes when the tensor does
                self._maps[index] = None
            if self._handles[index] is not None:
                self._handles[index].close()
                self._handles[index] = None


def write_safetensors(path: str, tensors: dict) -> None:
    """Write `tensors` (name -> CPU torch tensor) as one safetensors file, in the given order."""
    header = {}
    cursor = 0
    for name, tensor in tensors.items():
        if tensor.dtype not in _NAMES:
            raise SafetensorsError(f"cannot store tensor {name!r} of dtype {tensor.dtype}")
        size = tensor.numel() * tensor.element_size()
        header[name] = {"dtype": _NAMES[tensor.dtype], "shape": list(tensor.shape),
                        "data_offsets": [cursor, cursor + size]}
        cursor += size
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((8 - len(raw) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as handle:
        handle.write(struct.pack("<Q", len(raw)))
        handle.write(raw)
        for tensor in tensors.values():
            data = tensor.detach().contiguous().cpu()
            if data.numel():
                handle.write(data.view(torch.uint8).numpy().tobytes() if data.dim() else
                             data.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)
