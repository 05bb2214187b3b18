"""How the parts of a layer are arranged.

``PreNormBlock`` is the reference's Llama block (fms/models/llama.py:137-162):
  h = x + mixer(norm1(x));  y = h + feed_forward(norm2(h)).
The residual stream is float32.  A branch's output is not added at once: it is
left pending and the next norm kernel adds it while it reads the stream, so the
sum is formed in float32 and the stream is read and written once per branch.
"""

from __future__ import annotations

from typing import Optional

import torch

from .base import Part, register_part


class ResidualStream:
    """The float32 stream [T, width] and the branch output still to be added to it."""

    def __init__(self, resid: torch.Tensor):
        self.resid = resid
        self.pending: Optional[torch.Tensor] = None


class PreNormBlock(Part):
    def __init__(self, mixer: Part, feed_forward: Part, norm1: Part, norm2: Part,
                 names=("ln", "attn", "ff_ln", "ff_sub_layer")):
        super().__init__()
        self.norm1 = self.add_child(names[0], norm1)
        self.mixer = self.add_child(names[1], mixer)
        self.norm2 = self.add_child(names[2], norm2)
        self.feed_forward = self.add_child(names[3], feed_forward)

    def forward(self, stream: ResidualStream, batch, cache, act_dtype: torch.dtype) -> None:
        h = self.norm1.add_norm(stream.resid, stream.pending, act_dtype)
        stream.pending = self.mixer.forward(h, batch, cache)
        h = self.norm2.add_norm(stream.resid, stream.pending, act_dtype)
        stream.pending = self.feed_forward.forward(h)


register_part("block", "pre_norm", PreNormBlock)
