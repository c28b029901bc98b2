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
        self.pending_norm: Optional[Part] = None  # the norm that the pending branch passes before it is added
        self.prepared: Optional[tuple] = None  # (norm, NormedRows) of the stream as it is now

    def normed(self, norm: Part, act_dtype: torch.dtype, deferred_ok: bool = False, rows: Optional[torch.Tensor] = None):
        """The stream (with what is pending added) through `norm`: a tensor, or a NormedRows if allowed and at hand."""
        prepared, self.prepared = self.prepared, None
        if prepared is not None and prepared[0] is norm and deferred_ok and rows is None and self.fuse_products:
            return prepared[1]
        pending, self.pending = self.pending, None
        pending_norm, self.pending_norm = self.pending_norm, None
        if pending_norm is not None:
            return norm.add_norm(self.resid, pending, act_dtype, rows, branch_norm=pending_norm)
        return norm.add_norm(self.resid, pending, act_dtype, rows)

    def add_branch(self, out, next_norm: Optional[Part] = None, post_norm: Optional[Part] = None) -> None:
        """Takes a branch's output: a tensor (added when the stream is next read) or a BranchOutput.  post_norm: the
        branch joins the stream through that norm (the norm that reads the stream next applies both)."""
        if self.pending is not None:
            raise RuntimeError("a branch output is still to be added: read the stream through a norm between two branches")
        if post_norm is not None:
            # the branch's norm needs the whole row of the branch: its last product cannot add into the stream
            self.pending = out.value() if isinstance(out, BranchOutput) else out
            self.pending_norm = post_norm
            self.prepared = None
            return
        if isinstance(out, BranchOutput):
            lin = out.linear
            if (self.fuse_products and next_norm is not None and getattr(next_norm, "deferrable", lambda: False)()
                    and getattr(lin, "streams", lambda *a: False)(out.x.shape[0], out.x.dtype)
                    and self.resid.shape[1] == lin.out_features):
                scale = next_norm.scale_weight() if hasattr(next_norm, "scale_weight") else next_norm.w.get("weight")
                scaled, row_norm = ops.linear_into_stream(out.x, lin.w["weight"], lin.w.get("bias"), self.resid, scale, next_norm.eps)
                self.prepared = (next_norm, NormedRows(scaled, row_norm))
                return
            out = out.value()
        self.pending = out
        self.prepared = None


class PreNormBlock(Part):
    fuses_next_norm = True  # forward takes the norm that reads the stream after this block
    norm_arguments = ("norm1", "norm2")  # the norms the block is built with, by constructor argument

    def __init__(self, mixer: Part, feed_forward: Optional[Part], norm1: Part, norm2: Part,
                 names=("ln", "attn", "ff_ln", "ff_sub_layer")):
        """The feed-forward may be absent (None): the block is then its mixer branch alone, and has no second norm."""
        super().__init__()
        self.norm1 = self.add_child(names[0], norm1)
        self.mixer = self.add_child(names[1], mixer)
        self.feed_forward = feed_forward
        if feed_forward is not None:
            self.norm2 = self.add_child(names[2], norm2)
            self.add_child(names[3], feed_forward)

    def first_norm(self) -> Part:
        return self.norm1

    def forward(self, stream: ResidualStream, batch, cache, act_dtype: torch.dtype, next_norm: Optional[Part] = None) -> None:
        T = stream.resid.shape[0]
        mixer_takes = getattr(self.mixer, "accepts_normed_rows", None)
        h = stream.normed(self.norm1, act_dtype, mixer_takes is not None and mixer_takes(T, act_dtype, batch))
        branch = getattr(self.mixer, "forward_branch", self.mixer.forward)
        if self.feed_forward is None:
            stream.add_branch(branch(h, batch, cache), next_norm)
            return
        stream.add_branch(branch(h, batch, cache), self.norm2)
        ff_takes = getattr(self.feed_forward, "accepts_normed_rows", None)
        h = stream.normed(self.norm2, act_dtype, ff_takes is not None and ff_takes(T, act_dtype))
        branch = getattr(self.feed_forward, "forward_branch", self.feed_forward.forward)
        stream.add_branch(branch(h), next_norm)


class SandwichNormBlock(Part):
    """A block whose branches are normed on both sides: h = x + norm1b(mixer(norm1(x))); y = h + norm2b(ff(norm2(h))).
    The feed-forward may be absent (None): the block is then its mixer branch alone.  The norm behind a branch, the
    residual sum and the norm in front of the next branch are one kernel."""

    norm_arguments = ("norm1", "norm1b", "norm2", "norm2b")

    def __init__(self, mixer: Part, feed_forward: Optional[Part], norm1: Part, norm1b: Part, norm2: Part, norm2b: Part,
                 names=("norm1", "mix", "norm1b", "norm2", "mlp", "norm2b")):
        super().__init__()
        self.norm1 = self.add_child(names[0], norm1)
        self.mixer = self.add_child(names[1], mixer)
        self.norm1b = self.add_child(names[2], norm1b)
        self.feed_forward = feed_forward
        if feed_forward is not None:
            self.norm2 = self.add_child(names[3], norm2)
            self.add_child(names[4], feed_forward)
            self.norm2b = self.add_child(names[5], norm2b)

    def first_norm(self) -> Part:
        return self.norm1

    def forward(self, stream: ResidualStream, batch, cache, act_dtype: torch.dtype, next_norm: Optional[Part] = None) -> None:
        h = stream.normed(self.norm1, act_dtype)
        stream.add_branch(self.mixer.forward(h, batch, cache), post_norm=self.norm1b)
        if self.feed_forward is not None:
            h = stream.normed(self.norm2, act_dtype)
            stream.add_branch(self.feed_forward.forward(h), post_norm=self.norm2b)


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
