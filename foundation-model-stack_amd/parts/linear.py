"""A linear layer y = x W^T (+ b) with the weight stored [out, in] as checkpoints store it
(fms/modules/linear.py:254-255: the reference's only linear type on this path is nn.Linear)."""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Part


class Linear(Part):
    def __init__(self, in_features: int, out_features: int, bias: bool = False):
        super().__init__()
        self.in_features, self.out_features, self.has_bias = in_features, out_features, bias
        self.declare("weight", (out_features, in_features))
        if bias:
            self.declare("bias", (out_features,), init="zeros")

    def forward(self, x: torch.Tensor, out_dtype: Optional[torch.dtype] = None, row_norm=None) -> torch.Tensor:
        return ops.linear(x, self.w["weight"], self.w.get("bias"), out_dtype=out_dtype, row_norm=row_norm)

    def streams(self, rows: int, dtype: torch.dtype) -> bool:
        """True if a product of this shape runs in the weight-streaming kernel, which can take a deferred
        row norm on its input and add its output into the residual stream."""
        return dtype == torch.bfloat16 and self.w["weight"].dtype == torch.bfloat16 and rows <= ops.SKINNY_FAST_ROWS \
            and self.in_features % 8 == 0
