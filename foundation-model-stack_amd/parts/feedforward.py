"""Feed-forward parts.

``GatedLinearUnit`` is the reference's SwiGLU (fms/modules/feedforward.py:193-327):
one fused projection whose first half is the gate and second half the "up" path
(:288-297), out = w2(act(gate) * up).
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import BranchOutput, FeedForward, register_part, split_normed
from .linear import Linear


class GatedLinearUnit(FeedForward):
    def __init__(self, width: int, hidden_dim: int, activation: str = "swish", use_bias: bool = False):
        super().__init__()
        activation = str(activation).lower()  # the reference looks names up without regard to case
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(ops.ACTIVATIONS)}")
        self.width, self.hidden_dim, self.activation = width, int(hidden_dim), activation
        self.wg1 = self.add_child("wg1_fused", Linear(width, 2 * self.hidden_dim, use_bias))
        self.w2 = self.add_child("w2", Linear(self.hidden_dim, width, use_bias))

    def unfused_parameters(self) -> dict:
        """fms/modules/feedforward.py:312-327: the gate rows come first, then the "up" rows."""
        return {"wg1_fused": (("wg", self.hidden_dim), ("w1", self.hidden_dim))}

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.forward_branch(x).value()

    def accepts_normed_rows(self, rows: int, dtype) -> bool:
        return self.wg1.streams(rows, dtype)

    def forward_branch(self, x) -> BranchOutput:
        x, row_norm = split_normed(x)
        hidden = ops.gated_linear(x, self.wg1.w["weight"], self.wg1.w.get("bias"), self.activation, row_norm=row_norm)
        return BranchOutput(hidden, self.w2)


register_part("feed_forward", "glu", GatedLinearUnit)
