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
        weight_offset: float = 0.0,
        groups: int = 1,
    ):
        """weight_offset: the stored weight is the scale minus this number (1.0 for a scale stored around zero); the sum
        is formed once, in float32, when the model is finalized.
        groups: the row is split into that many equal consecutive parts, each divided by its own root mean square
        (RMS norms without a shift only); the weight covers the whole row."""
        super().__init__()
        self.width, self.eps, self.use_mean = width, float(eps), use_mean
        self.groups = int(groups)
        if self.groups < 1 or width % self.groups:
            raise ValueError(f"{groups} groups do not divide a width of {width}")
        if self.groups > 1 and (use_mean or elementwise_shift):
            raise ValueError("a norm in groups is an RMS norm: no mean, no shift")
        self.weight_offset = float(weight_offset)
        self._scale: Optional[torch.Tensor] = None
        if elementwise_scale:
            # random-weights mode gives a scale of one either way
            self.declare("weight", (width,), init="ones" if self.weight_offset == 0.0 else "zeros", kind="scale")
        if elementwise_shift:
            self.declare("bias", (width,), init="zeros", kind="scale")

    def finalize(self, device, dtype) -> None:
        if self.weight_offset and self.w.get("weight") is not None:
            self._scale = (self.w["weight"].to(torch.float32) + self.weight_offset).contiguous()

    def scale_weight(self) -> Optional[torch.Tensor]:
        """The scale that multiplies the normed rows: the stored weight, plus its offset if it has one."""
        return self._scale if self._scale is not None else self.w.get("weight")

    def add_norm(
        self,
        resid: torch.Tensor,
        branch: Optional[torch.Tensor],
        out_dtype: torch.dtype,
        rows: Optional[torch.Tensor] = None,
        branch_norm: Optional["ParameterizedNorm"] = None,
    ) -> torch.Tensor:
        """resid += branch (float32, in place); returns norm(resid) in out_dtype (only `rows` if given).
        branch_norm: the branch goes through that norm first (a block that norms its branches before they join the
        stream); both norms and the sum are then one kernel."""
        grouped = self.groups > 1 or (branch_norm is not None and branch_norm.groups > 1)
        if grouped:
            if not self._plain_rms() or (branch_norm is not None and not branch_norm._plain_rms()):
                raise NotImplementedError("norms in groups are RMS norms without mean and shift")
            return ops.group_norm_chain(resid, branch, branch_norm.scale_weight() if branch_norm is not None else None,
                                        branch_norm.groups if branch_norm is not None else 0,
                                        branch_norm.eps if branch_norm is not None else 0.0, out_dtype, ops.CHAIN_NORM,
                                        self.scale_weight(), self.groups, self.eps, rows)
        if branch_norm is not None and branch is not None:
            if not (self.deferrable() and branch_norm.deferrable()):
                # norms that take the mean off or add a shift (layer norms): the general chain
                vectors = [branch_norm.scale_weight(), branch_norm.w.get("bias"), self.scale_weight(), self.w.get("bias")]
                if len({v.dtype for v in vectors if v is not None}) > 1:
                    vectors = [v.to(torch.float32) if v is not None else None for v in vectors]  # the kernel takes one type
                return ops.norm_add_norm_affine(resid, branch, vectors[0], vectors[1], branch_norm.eps, branch_norm.use_mean,
                                                vectors[2], vectors[3], self.eps, self.use_mean, out_dtype, rows)
            return ops.norm_add_norm(resid, branch, branch_norm.scale_weight(), branch_norm.eps, self.scale_weight(), self.eps,
                                     out_dtype, rows)
        bias = self.w.get("bias")
        if bias is not None and self._scale is not None:
            bias = bias.to(torch.float32)  # the kernel takes scale and shift of one type
        return ops.add_norm(resid, branch, self.scale_weight(), bias, self.eps, out_dtype, rows, self.use_mean)

    def join(self, resid: torch.Tensor, branch: torch.Tensor, act_dtype: torch.dtype, want_rows: bool) -> Optional[torch.Tensor]:
        """resid += norm(branch) (float32, in place), for a block whose norms sit behind its branches; returns the stream
        in act_dtype if `want_rows` (what the next branch reads: the stream itself, not normed)."""
        if not self._plain_rms():
            raise NotImplementedError("a branch joins the stream through an RMS norm without mean and shift")
        return ops.group_norm_chain(resid, branch, self.scale_weight(), self.groups, self.eps, act_dtype,
                                    ops.CHAIN_CAST if want_rows else ops.CHAIN_NONE)

    def _plain_rms(self) -> bool:
        return not self.use_mean and "bias" not in self.w

    def deferrable(self) -> bool:
        """True if the norm is a row scale times a weight (no mean, no shift, one group), so that a product can apply the
        row scale to its result instead: (x / rms(x) * w) W^T = (x * w) W^T / rms(x)."""
        return self._plain_rms() and self.groups == 1


register_part("norm", "rmsnorm", lambda width, eps=1e-6, **kw: ParameterizedNorm(width, eps, True, False, False, **kw))
register_part("norm", "layernorm", lambda width, eps=1e-6, **kw: ParameterizedNorm(width, eps, True, True, True, **kw))
register_part("norm", "parameterized", ParameterizedNorm)
