"""The parameterised norm of the reference (fms/modules/layernorm.py:5-69).

Llama uses it as RMSNorm: no mean subtraction, a learned scale, no shift, eps
inside the root.  Statistics, scaling and the multiplication by the weight are
float32; the result is rounded once to the activation type.  The kernel also
folds in the residual addition that precedes the norm in a pre-norm block.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import Part, register_part


class ParameterizedNorm(Part):
    def __init__(
        self,
        width: int,
        eps: float = 1e-6,
        elementwise_scale: bool = True,
        elementwise_shift: bool = False,
        use_mean: bool = False,
    ):
        super().__init__()
        self.width, self.eps, self.use_mean = width, float(eps), use_mean
        if elementwise_scale:
            self.declare("weight", (width,), init="ones", kind="scale")
        if elementwise_shift:
            self.declare("bias", (width,), init="zeros", kind="scale")

    def add_norm(
        self,
        resid: torch.Tensor,
        branch: Optional[torch.Tensor],
        out_dtype: torch.dtype,
        rows: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        """resid += branch (float32, in place); returns norm(resid) in out_dtype (only `rows` if given)."""
        return ops.add_norm(resid, branch, self.w.get("weight"), self.w.get("bias"), self.eps, out_dtype, rows, self.use_mean)

    def deferrable(self) -> bool:
        """True if the norm is a row scale times a weight (no mean, no shift), so that a product can apply the
        row scale to its result instead: (x / rms(x) * w) W^T = (x * w) W^T / rms(x)."""
        return not self.use_mean and "bias" not in self.w


register_part("norm", "rmsnorm", lambda width, eps=1e-6, **kw: ParameterizedNorm(width, eps, True, False, False, **kw))
register_part("norm", "layernorm", lambda width, eps=1e-6, **kw: ParameterizedNorm(width, eps, True, True, True, **kw))
register_part("norm", "parameterized", ParameterizedNorm)
