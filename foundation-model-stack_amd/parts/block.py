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

from ..cache import StateNeed
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

    def rows(self, act_dtype: torch.dtype, want_rows: bool = True) -> Optional[torch.Tensor]:
        """The stream itself, not normed, with what is pending added: in the activation type if `want_rows` (in a
        float32 model the stream's own tensor), else nothing.  For blocks whose branches read the stream as it is."""
        self.prepared = None
        pending, self.pending = self.pending, None
        pending_norm, self.pending_norm = self.pending_norm, None
        if pending is not None and pending_norm is None:
            raise NotImplementedError("a branch without a norm of its own is added by the norm that reads the stream next")
        copy_wanted = want_rows and act_dtype != torch.float32
        if pending is not None:
            out = pending_norm.join(self.resid, pending, pending.dtype, copy_wanted)
        else:
            out = ops.cast(self.resid, act_dtype) if copy_wanted else None
        if not want_rows:
            return None
        return out if copy_wanted else self.resid

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


class PostNormBlock(Part):
    """A block whose norms sit behind its branches only: h = x + norm1(mixer(x')); y = h + norm2(ff(h)).  The branches read
    the stream itself.  With `input_taps` the mixer reads x' = x + conv(x), a causal convolution over time on every
    channel of the stream (weight [width, taps], no bias, the last column the token's own); the stream's last
    taps - 1 rows are then part of a sequence's state.  The feed-forward may be absent (None).  The norm behind a branch
    and the residual sum are one kernel, which also leaves what the next branch reads."""

    norm_arguments = ("norm1", "norm2")

    def __init__(self, mixer: Part, feed_forward: Optional[Part], norm1: Part, norm2: Part, width: int = 0, input_taps: int = 0,
                 names=("norm1", "mix", "norm2", "mlp", "canon1")):
        super().__init__()
        self.mixer = self.add_child(names[1], mixer)
        self.norm1 = self.add_child(names[0], norm1)
        self.feed_forward = feed_forward
        if feed_forward is not None:
            self.norm2 = self.add_child(names[2], norm2)
            self.add_child(names[3], feed_forward)
        self.input_taps = int(input_taps)
        self.width = int(width)
        self._conv_name = names[4]
        if self.input_taps:
            if not 1 <= self.input_taps <= ops.CONV_MAX_TAPS or self.width <= 0:
                raise ValueError(f"an input convolution of {input_taps} taps (1 to {ops.CONV_MAX_TAPS}) over {width} channels")
            self.declare(names[4], (self.width, self.input_taps))

    def state_need(self) -> Optional[StateNeed]:
        """The stream's last taps - 1 rows of every sequence (float32), under a name that no mixer's state has."""
        if self.input_taps > 1:
            return StateNeed((("block.conv", (self.input_taps - 1, self.width), "float32"),))
        return None

    def forward(self, stream: ResidualStream, batch, cache, act_dtype: torch.dtype, next_norm: Optional[Part] = None) -> None:
        if self.input_taps:
            x = stream.rows(torch.float32)
            h = ops.short_conv(x, 0, self.width, self.w[self._conv_name], None, cache.state.get("block.conv"), batch.seq_of_token,
                               batch.slot_ids, act_dtype, add_input=True, single_tokens=batch.is_decode)
        else:
            h = stream.rows(act_dtype)
        stream.add_branch(self.mixer.forward(h, batch, cache), post_norm=self.norm1)
        if self.feed_forward is not None:
            stream.add_branch(self.feed_forward.forward(stream.rows(act_dtype)), post_norm=self.norm2)


register_part("block", "pre_norm", PreNormBlock)
register_part("block", "post_norm", PostNormBlock)
register_part("block", "sandwich_norm", SandwichNormBlock)
