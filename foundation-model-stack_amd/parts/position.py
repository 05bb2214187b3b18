"""Position encodings.

``RotaryEncoding`` is the reference's RoPE without complex numbers
(fms/modules/positions.py:269-464): adjacent pairs (x[2i], x[2i+1]) are rotated
by position * f_i, f_i = theta^(-2i/D), all in float32.  The frequencies are
computed with the reference's own expression; the cos/sin table is built once
on the device by a kernel and read by the fused rotate-and-store kernel.

The interface a position encoding offers to a mixer:
  * ``rotary_tables()``: (cos, sin, rotary size) for the fused kernel, or None;
  * ``adjust_qk(qkv, batch, ...)``: transform queries and keys in place before
    they are cached, for encodings that are no plain rotation;
  * ``check_positions(max_position)``: raise if a position cannot be encoded.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from ..kernels import ops
from .base import Part, register_part


def rope_frequencies(dim: int, theta: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """Float32 frequencies f_i, i < dim/2.

    regular: fms/modules/positions.py:124-132.  llama3: fms/modules/positions.py:171-196.
    """
    scaling = dict(scaling or {})
    kind = scaling.get("rope_type", "regular")
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
    if kind == "regular":
        return freqs
    if kind == "llama3":
        factor = scaling["factor"]
        low_freq_factor = scaling["low_freq_factor"]
        high_freq_factor = scaling["high_freq_factor"]
        old_len = scaling["original_max_position_embeddings"]
        wavelen = 2 * math.pi / freqs
        scaled = torch.where(wavelen > old_len / low_freq_factor, freqs / factor, freqs)
        smooth = (old_len / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
        smoothed = (1 - smooth) * scaled / factor + smooth * scaled
        medium = ~(wavelen < old_len / high_freq_factor) * ~(wavelen > old_len / low_freq_factor)
        return torch.where(medium, smoothed, scaled)
    raise ValueError(f"rope_type {kind!r} is not supported (regular, llama3)")


class PositionEncoding(Part):
    def rotary_tables(self) -> Optional[Tuple[torch.Tensor, torch.Tensor, int]]:
        return None

    def adjust_qk(self, qkv: torch.Tensor, batch, nheads: int, kvheads: int, head_dim: int) -> None:
        """In-place transform of the query and key columns of qkv rows; default: none."""

    def check_positions(self, max_position: int) -> None:
        """Raise IndexError when `max_position` cannot be encoded."""


class RotaryEncoding(PositionEncoding):
    def __init__(self, dim: int, theta: float = 10_000.0, max_seq_len: int = 2048, scaling: Optional[dict] = None,
                 partial_rope: float = 1.0):
        super().__init__()
        self.head_dim = dim
        self.rot_dim = int(partial_rope * dim)
        if self.rot_dim % 2 or self.rot_dim <= 0 or self.rot_dim > dim:
            raise ValueError(f"rotary size {self.rot_dim} of head size {dim} must be even and within the head")
        self.theta, self.max_seq_len, self.scaling = float(theta), int(max_seq_len), dict(scaling or {})
        self.freqs = rope_frequencies(self.rot_dim, self.theta, self.scaling)
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def finalize(self, device, dtype) -> None:
        self.cos, self.sin = ops.rope_table(self.freqs.to(device), self.max_seq_len)

    def rotary_tables(self):
        return self.cos, self.sin, self.rot_dim

    def check_positions(self, max_position: int) -> None:
        # tests/modules/test_positions.py:156-168: a position beyond the table raises
        if max_position >= self.max_seq_len:
            raise IndexError(f"position {max_position} is beyond the rotary table of {self.max_seq_len} positions")


register_part("position", "rope", RotaryEncoding)
