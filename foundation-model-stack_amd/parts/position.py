"""Position encodings.

``RotaryEncoding`` is the reference's RoPE without complex numbers
(fms/modules/positions.py:269-464): adjacent pairs (x[2i], x[2i+1]) are rotated
by position * f_i, f_i = theta^(-2i/D), all in float32.  The frequencies are
computed with the reference's own expression; the cos/sin table is built once
on the device by a kernel and read by the fused rotate-and-store kernel.

The interface a position encoding offers to a mixer:
  * ``rotary_tables()``: (cos, sin, rotary size) for the fused kernel, or None;
    ``tables_for_step(batch)``: the same for one step, for encodings whose table depends on the step;
  * ``adjust_qk(qkv, batch, ...)``: transform queries and keys in place before
    they are cached, for encodings that are no plain rotation;
  * ``score_slopes(nheads)``: for encodings that act on the scores instead (the reference's
    ``adjusted_mask``, fms/modules/positions.py:9-36): a float32 slope per head, added to every score as
    slope * (key position - query position); None for encodings that leave the scores alone;
  * ``check_positions(max_position)``: raise if a position cannot be encoded.
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from ..kernels import ops
from .base import Part, register_part


def ntk_alpha(length: int, original_length: int) -> int:
    """fms/modules/positions.py:146-156: the power of two that stretches `original_length` over `length`."""
    ratio = max(1, -(-int(length) // int(original_length)))
    return 1 << (ratio - 1).bit_length()


def rope_frequencies(dim: int, theta: float, scaling: Optional[dict] = None, alpha: int = 1) -> torch.Tensor:
    """Float32 frequencies f_i, i < dim/2.

    regular: fms/modules/positions.py:124-132.  llama3: fms/modules/positions.py:171-196.
    ntk: fms/modules/positions.py:161-168, theta * alpha^(dim / (dim - 2)) for the power of two `alpha`.
    """
    scaling = dict(scaling or {})
    kind = scaling.get("rope_type", "regular")
    if kind == "ntk":
        theta = theta * alpha ** (dim / (dim - 2))
    freqs = 1.0 / (theta ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
    if kind in ("regular", "ntk"):
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
    raise ValueError(f"rope_type {kind!r} is not supported (regular, llama3, ntk)")


class PositionEncoding(Part):
    def rotary_tables(self) -> Optional[Tuple[torch.Tensor, torch.Tensor, int]]:
        return None

    def tables_for_step(self, batch) -> Optional[Tuple[torch.Tensor, torch.Tensor, int]]:
        """The tables for the tokens of one step; the same for every step unless the encoding says otherwise."""
        return self.rotary_tables()

    def adjust_qk(self, qkv: torch.Tensor, batch, nheads: int, kvheads: int, head_dim: int) -> None:
        """In-place transform of the query and key columns of qkv rows; default: none."""

    def score_slopes(self, nheads: int) -> Optional[torch.Tensor]:
        """float32 [nheads] on the device: a bias by distance that attention adds to its scores; default: none."""
        return None

    def check_positions(self, max_position: int) -> None:
        """Raise IndexError when `max_position` cannot be encoded."""


class RotaryEncoding(PositionEncoding):
    """max_seq_len: the length of the table (the reference's max_expected_seq_len).  With "ntk" scaling it is the
    length the frequencies were made for, and sequences may grow to `max_positions`: a step whose longest
    sequence holds n tokens rotates all its tokens with the table of alpha = ntk_alpha(n, max_seq_len), as
    the reference's call does (fms/modules/positions.py:311-355, 407-421: alpha from the call's longest
    sequence; keys cached by earlier calls keep the rotation they got).  Up to max_seq_len tokens alpha is 1 and
    the encoding is the regular one (tests/modules/test_positions.py:216-241)."""

    def __init__(self, dim: int, theta: float = 10_000.0, max_seq_len: int = 2048, scaling: Optional[dict] = None,
                 partial_rope: float = 1.0, max_positions: Optional[int] = None):
        super().__init__()
        self.head_dim = dim
        self.rot_dim = int(partial_rope * dim)
        if self.rot_dim % 2 or self.rot_dim <= 0 or self.rot_dim > dim:
            raise ValueError(f"rotary size {self.rot_dim} of head size {dim} must be even and within the head")
        self.theta, self.max_seq_len, self.scaling = float(theta), int(max_seq_len), dict(scaling or {})
        self.stretches = self.scaling.get("rope_type") == "ntk"
        self.max_positions = int(max_positions) if (max_positions and self.stretches) else self.max_seq_len
        if self.stretches and self.rot_dim <= 2:
            raise ValueError("ntk scaling needs a rotary size above 2")
        self.freqs = rope_frequencies(self.rot_dim, self.theta, self.scaling)
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None
        self.tables = {}  # alpha -> (cos, sin); alpha 1 only unless the encoding stretches

    @property
    def graph_safe(self) -> bool:
        """A captured step keeps the tables it was captured with; a stretching encoding changes them as sequences grow."""
        return self.max_positions <= self.max_seq_len

    def finalize(self, device, dtype) -> None:
        alpha = 1
        while True:
            length = min(self.max_seq_len * alpha, self.max_positions)
            freqs = rope_frequencies(self.rot_dim, self.theta, self.scaling, alpha)
            self.tables[alpha] = ops.rope_table(freqs.to(device), length)
            if self.max_seq_len * alpha >= self.max_positions:
                break
            alpha *= 2
        self.cos, self.sin = self.tables[1]

    def rotary_tables(self):
        return self.cos, self.sin, self.rot_dim

    def tables_for_step(self, batch):
        if not self.stretches:
            return self.cos, self.sin, self.rot_dim
        cos, sin = self.tables[ntk_alpha(batch.max_context, self.max_seq_len)]
        return cos, sin, self.rot_dim

    def check_positions(self, max_position: int) -> None:
        # tests/modules/test_positions.py:156-168: a position beyond the table raises
        if max_position >= self.max_positions:
            raise IndexError(f"position {max_position} is beyond the rotary table of {self.max_positions} positions")


register_part("position", "rope", RotaryEncoding)
