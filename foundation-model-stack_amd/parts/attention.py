"""Multi-head attention with grouped kv heads over the paged cache: the mixer of Llama.

The reference's order of operations (fms/modules/attention.py:870-937): one fused
projection split into [H*D | K*D | K*D]; rotate queries and keys; append keys and
values to the cache; causal scaled-dot-product attention in which query head h reads
kv head h // (H/K) (:241-250) with scale 1/sqrt(D) unless given (:768-784); output
projection.  Here the rotation and the cache append are one kernel, and attention
reads the cache directly, so a step may bring any number of new tokens per sequence.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from ..cache import KVNeed
from ..kernels import ops
from .base import BranchOutput, Mixer, Part, register_part, split_normed
from .linear import Linear
from .position import PositionEncoding


class LayerCache:
    """What a mixer sees of the cache for one schedule entry."""

    def __init__(self, group: int, keys: Optional[torch.Tensor], values: Optional[torch.Tensor], owns: bool, state: dict):
        self.group, self.keys, self.values, self.owns, self.state = group, keys, values, owns, state


class MultiHeadAttention(Mixer):
    def __init__(
        self,
        width: int,
        nheads: int,
        kvheads: int,
        head_dim: int,
        use_bias: bool = False,
        position_encoder: Optional[PositionEncoding] = None,
        scale_factor: Optional[float] = None,
        window: int = 0,
        soft_cap: float = 0.0,
    ):
        super().__init__()
        if kvheads <= 0 or nheads % kvheads:
            raise ValueError(f"{nheads} query heads are no multiple of {kvheads} kv heads")
        if head_dim % 2 or head_dim > 256:
            raise ValueError(f"head size {head_dim} must be even and at most 256")
        self.width, self.nheads, self.kvheads, self.head_dim = width, nheads, kvheads, head_dim
        self.scale = float(scale_factor) if scale_factor is not None else 1.0 / math.sqrt(head_dim)
        self.window = int(window)
        self.soft_cap = float(soft_cap)  # scores become soft_cap * tanh(score / soft_cap); 0: no cap
        if self.soft_cap < 0:
            raise ValueError(f"soft_cap {soft_cap} must be zero (none) or positive")
        self.position_encoder = position_encoder
        in_proj = self.add_child("in_proj", Part())
        self.qkv = in_proj.add_child("qkv_fused", Linear(width, (nheads + 2 * kvheads) * head_dim, use_bias))
        self.dense = self.add_child("dense", Linear(nheads * head_dim, width, use_bias))

    def unfused_parameters(self) -> dict:
        """The fused projection as the parts it is made of: fused local name -> ((local name, rows), ...), in the
        order of the rows (fms/modules/attention.py:666-687)."""
        H, K, D = self.nheads, self.kvheads, self.head_dim
        return {"in_proj.qkv_fused": (("in_proj.query", H * D), ("in_proj.key", K * D), ("in_proj.value", K * D))}

    # ---- what the mixer asks of the cache ---------------------------------
    def kv_need(self) -> Optional[KVNeed]:
        return KVNeed(self.kvheads, self.head_dim, self.window)

    def state_need(self):
        return None

    @property
    def graph_safe(self) -> bool:
        return getattr(self.position_encoder, "graph_safe", True)

    def check_step(self, max_position: int) -> None:
        if self.position_encoder is not None:
            self.position_encoder.check_positions(max_position)

    def _score_slopes(self) -> Optional[torch.Tensor]:
        return self.position_encoder.score_slopes(self.nheads) if self.position_encoder is not None else None

    def prefill_qblock(self, n_tokens: int, dtype) -> int:
        if dtype != torch.bfloat16 or self.head_dim % 16 or self.soft_cap > 0 or self._score_slopes() is not None:
            return 0  # the generic kernel takes tokens one by one
        return ops.prefill_qblock(self.nheads, self.kvheads, self.head_dim, n_tokens)

    def _fused_decode(self, rows: int, dtype, batch) -> bool:
        """True if projection, rotation and cache write of this step run as one kernel."""
        rotates_by_table = self.position_encoder is None or self.position_encoder.rotary_tables() is not None
        return (batch.is_decode and rows <= ops.QKV_ROPE_MAX_ROWS and dtype == torch.bfloat16
                and self.qkv.w["weight"].dtype == torch.bfloat16 and self.head_dim % 16 == 0 and self.width % 8 == 0
                and rotates_by_table)

    def accepts_normed_rows(self, rows: int, dtype, batch) -> bool:
        return self._fused_decode(rows, dtype, batch)

    def forward(self, x: torch.Tensor, batch, cache: LayerCache) -> torch.Tensor:
        return self.forward_branch(x, batch, cache).value()

    def forward_branch(self, x, batch, cache: LayerCache) -> BranchOutput:
        x, row_norm = split_normed(x)
        H, K, D = self.nheads, self.kvheads, self.head_dim
        table = batch.block_tables[cache.group]
        tables = self.position_encoder.tables_for_step(batch) if self.position_encoder is not None else None
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        keys, values = (cache.keys, cache.values) if cache.owns else (None, None)
        weight = self.qkv.w["weight"]
        if self._fused_decode(x.shape[0], x.dtype, batch):
            # decode: projection, rotation and cache write in one kernel
            qkv = ops.qkv_rope_write(x, weight, self.qkv.w.get("bias"), batch.positions, batch.seq_of_token, table,
                                     cos, sin, rot, keys, values, H, K, D, row_norm=row_norm)
        else:
            if row_norm is not None:
                raise RuntimeError("a deferred norm reached a step that does not take one")
            qkv = self.qkv.forward(x)
            if tables is None and self.position_encoder is not None:
                self.position_encoder.adjust_qk(qkv, batch, H, K, D)
            ops.rope_kv_write(qkv, batch.positions, batch.seq_of_token, table, cos, sin, rot, keys, values, H, K, D)
        size = 0 if batch.is_decode else self.prefill_qblock(batch.n_tokens, x.dtype)
        qb_start, qb_len = batch.qblocks.get(size, (None, None))
        mixed = ops.attention(
            qkv, batch.positions, batch.seq_of_token, table, cache.keys, cache.values, H, K, D, self.scale, self.window,
            decode=batch.is_decode, max_context=batch.context_bound,
            qblock_start=qb_start, qblock_len=qb_len, qblock_tokens=size,
            row_order=batch.rows_by_length if batch.is_decode else None,
            score_slopes=self._score_slopes(), soft_cap=self.soft_cap,
        )
        return BranchOutput(mixed, self.dense)


register_part("mixer", "attention", MultiHeadAttention)
