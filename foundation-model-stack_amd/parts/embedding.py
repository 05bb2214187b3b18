"""Token embedding and output head.

fms/models/llama.py:185-187, 332: a table row per token, no scale.  The head is a
bias-free linear layer (fms/modules/head.py:89-95) whose logits leave in float32.
"""

from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, register_part


class TokenEmbedding(Part):
    def __init__(self, vocab: int, width: int):
        super().__init__()
        self.vocab, self.width = vocab, width
        self.declare("weight", (vocab, width))

    def forward(self, token_ids: torch.Tensor, batch=None) -> torch.Tensor:
        """int32 ids [T] -> the float32 residual stream [T, width].  `batch` is the step (positions, sequence of
        every token): an embedding that adds a learned vector per position reads it, this one does not."""
        return ops.embed(token_ids, self.w["weight"])


class LinearHead(Part):
    def __init__(self, width: int, vocab: int):
        super().__init__()
        self.vocab, self.width = vocab, width
        self.declare("weight", (vocab, width))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.linear(x, self.w["weight"], None, out_dtype=torch.float32)


register_part("embedding", "table", TokenEmbedding)
register_part("head", "linear", LinearHead)
