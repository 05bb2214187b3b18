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

from ..kernels import ops
from .base import BranchOutput, NormedRows, Part, register_part


class ResidualStream:
    """The float32 stream [T, width] and the branch output still to be added to it.

    In a decode step of few rows the branch's last product can add to the stream itself and leave the next
    norm's input behind (`prepared`), which the next branch's first product finishes: two kernels fewer per
    branch.  That is decided here, from what the parts say they can do; a part that says nothing gets a
    normed tensor and returns a tensor."""

    fuse_products = True  # class-wide switch: False keeps every norm a kernel of its own

    def __init__(self, resid: torch.Tensor):
        self.resid = resid
        self.pending: Optional[torch.Tensor] = None
        self.prepared: Optional[tuple] = None  # (norm, NormedRows) of the stream as it is now

    def normed(self, norm: Part, act_dtype: torch.dtype, deferred_ok: bool = False, rows: Optional[torch.Tensor] = None):
        """The stream (with what is pending added) through `norm`: a tensor, or a NormedRows if allowed and at hand."""
        prepared, self.prepared = self.prepared, None
        if prepared is not None and prepared[0] is norm and deferred_ok and rows is None and self.fuse_products:
            return prepared[1]
        pending, self.pending = self.pending, None
        return norm.add_norm(self.resid, pending, act_dtype, rows)

    def add_branch(self, out, next_norm: Optional[Part] = None) -> None:
        """Takes a branch's output: a tensor (added when the stream is next read) or a BranchOutput."""
        if self.pending is not None:
            raise RuntimeError("a branch output is still to be added: read the stream through a norm between two branches")
        if isinstance(out, BranchOutput):
            lin = out.linear
            if (self.fuse_products and next_norm is not None and getattr(next_norm, "deferrable", lambda: False)()
                    and getattr(lin, "streams", lambda *a: False)(out.x.shape[0], out.x.dtype)
                    and self.resid.shape[1] == lin.out_features):
                scaled, row_norm = ops.linear_into_stream(out.x, lin.w["weight"], lin.w.get("bias"), self.resid,
                                                          next_norm.w.get("weight"), next_norm.eps)
                self.prepared = (next_norm, NormedRows(scaled, row_norm))
                return
            out = out.value()
        self.pending = out
        self.prepared = None


class PreNormBlock(Part):
    fuses_next_norm = True  # forward takes the norm that reads the stream after this block
    norm_arguments = ("norm1", "norm2")  # the norms the block is built with, by constructor argument

    def __init__(self, mixer: Part, feed_forward: Part, norm1: Part, norm2: Part,
                 names=("ln", "attn", "ff_ln", "ff_sub_layer")):
        super().__init__()
        self.norm1 = self.add_child(names[0], norm1)
        self.mixer = self.add_child(names[1], mixer)
        self.norm2 = self.add_child(names[2], norm2)
        self.feed_forward = self.add_child(names[3], feed_forward)

    def first_norm(self) -> Part:
        return self.norm1

    def forward(self, stream: ResidualStream, batch, cache, act_dtype: torch.dtype, next_norm: Optional[Part] = None) -> None:
        T = stream.resid.shape[0]
        mixer_takes = getattr(self.mixer, "accepts_normed_rows", None)
        h = stream.normed(self.norm1, act_dtype, mixer_takes is not None and mixer_takes(T, act_dtype, batch))
        branch = getattr(self.mixer, "forward_branch", self.mixer.forward)
        stream.add_branch(branch(h, batch, cache), self.norm2)
        ff_takes = getattr(self.feed_forward, "accepts_normed_rows", None)
        h = stream.normed(self.norm2, act_dtype, ff_takes is not None and ff_takes(T, act_dtype))
        branch = getattr(self.feed_forward, "forward_branch", self.feed_forward.forward)
        stream.add_branch(branch(h), next_norm)


register_part("block", "pre_norm", PreNormBlock)
