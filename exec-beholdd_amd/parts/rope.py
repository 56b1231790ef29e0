"""Rotary position encoding, split-half pairing.

freq[i] = 1 / theta^(2i/rotary) for i < rotary/2, angle = position * freq[i]
(crates/beholdd-model/src/qwen3moe/forward.rs:1844-1868): powers, angles, cosines and sines are
computed in float64 and stored as float32, one row per position, once per model, like the
reference's device path (crates/beholdd-model/src/recorded_attention.rs:438-457).  The pairs
are (x[i], x[i + rotary/2]) (crates/beholdd-kernel/src/vecops.rs:186-197); the attention
kernel applies them.
"""

from __future__ import annotations

import numpy as np
import torch

from .base import POSITION_ENCODINGS


class RotaryEncoding:
    def __init__(self, rotary_dim: int, theta: float, max_position: int):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise ValueError(f"rotary width must be positive and even, got {rotary_dim}")
        if not (theta > 0.0):
            raise ValueError(f"RoPE base must be positive and finite, got {theta}")
        self.rotary_dim, self.theta, self.max_position = int(rotary_dim), float(theta), int(max_position)
        self._tables = None

    def tensor_specs(self):
        return []

    def load(self, get):
        pass

    def build_tables(self, device):
        half = self.rotary_dim // 2
        freqs = np.array([1.0 / (self.theta ** ((2 * i) / self.rotary_dim)) for i in range(half)], dtype=np.float64)
        angles = np.arange(self.max_position, dtype=np.float64)[:, None] * freqs[None, :]
        cos = torch.from_numpy(np.cos(angles).astype(np.float32)).to(device).contiguous()
        sin = torch.from_numpy(np.sin(angles).astype(np.float32)).to(device).contiguous()
        self._tables = (cos, sin)

    def tables(self):
        if self._tables is None:
            raise RuntimeError("rotary tables were not built; call build_tables(device) after loading")
        return self._tables


class NoPositionEncoding:
    """For mixers whose order information comes from elsewhere (or nowhere)."""

    def tensor_specs(self):
        return []

    def load(self, get):
        pass

    def build_tables(self, device):
        pass

    def tables(self):
        return (None, None)


@POSITION_ENCODINGS.register("rope")
def _build_rope(config, shared):
    return RotaryEncoding(config.head_dim, config.rope_theta, config.max_position)


@POSITION_ENCODINGS.register("none")
def _build_none(config, shared):
    return NoPositionEncoding()
