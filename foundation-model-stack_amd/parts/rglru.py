"""The real-gated linear recurrent unit inside a two-branch recurrent block: a mixer whose memory is one number per
channel instead of a cache of keys and values.

Both branches read the mixer's input h and have `channels` outputs: y = act(W_y h + b_y), and u = conv(W_x h + b_x), a
short causal convolution over time on every channel (with a bias, no activation).  u is cut into `blocks` equal parts;
inside each, two square matrices make the gates,

    r = sigmoid(Ra u + ba),   i = sigmoid(Ri u + bi),   log a = -c r softplus(lam),   a = exp(log a)
    S <- a S + sqrt(1 - a^2) (i u)                       from S = 0, also for a sequence's first token

and the block's output is W_o (S * y).  What a sequence carries from token to token is S (float32) and the last
`conv - 1` inputs of the convolution; both are fixed-size state of its slot, so whole prompts, portions of prompts and
single tokens start from the same numbers and differ by rounding only (long steps walk the recurrence in chunks of rows
side by side, which adds in another order).  Everything behind the projection is float32.
"""

from __future__ import annotations

import torch

from ..cache import StateNeed
from ..kernels import ops
from .base import BranchOutput, Mixer, register_part
from .linear import Linear


class RecurrentGatedUnit(Mixer):
    def __init__(self, width: int, channels: int, blocks: int, conv: int = 4, decay_constant: float = 8.0,
                 activation: str = "gelu-tanh", position_encoder=None):  # takes no positions: the recurrence knows its order
        super().__init__()
        if channels <= 0 or blocks <= 0 or channels % blocks:
            raise ValueError(f"{channels} channels do not split into {blocks} equal blocks")
        if not 1 <= conv <= ops.CONV_MAX_TAPS:
            raise ValueError(f"a convolution of {conv} taps (1 to {ops.CONV_MAX_TAPS})")
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {sorted(ops.ACTIVATIONS)}")
        self.width, self.channels, self.blocks, self.taps = width, int(channels), int(blocks), int(conv)
        self.decay_constant, self.activation = float(decay_constant), activation
        n = self.channels // self.blocks
        # one product for both branches: [y | x], with their biases
        self.in_proj = self.add_child("in_proj", Linear(width, 2 * self.channels, bias=True))
        self.declare("conv.weight", (self.channels, self.taps))
        self.declare("conv.bias", (self.channels,), init="zeros")
        self.declare("ra.weight", (self.blocks, n, n))
        self.declare("ra.bias", (self.blocks, n), init="zeros", kind="scale")
        self.declare("ri.weight", (self.blocks, n, n))
        self.declare("ri.bias", (self.blocks, n), init="zeros", kind="scale")
        self.declare("lam", (self.channels,), init="zeros", kind="scale")
        self.out = self.add_child("out", Linear(self.channels, width))
        self._ra_t = self._ri_t = self._ra_b = self._ri_b = self._lam = None

    def unfused_parameters(self) -> dict:
        return {"in_proj": (("y", self.channels), ("x", self.channels))}

    def state_need(self) -> StateNeed:
        tensors = [("S", (self.channels,), "float32")]
        if self.taps > 1:
            tensors.append(("conv", (self.taps - 1, self.channels), "float32"))
        return StateNeed(tuple(tensors))

    def output_projection(self) -> Linear:
        return self.out

    def finalize(self, device, dtype) -> None:
        # every block's matrix transposed, [in][out]: neighbouring threads of the gate kernel read neighbouring weights
        self._ra_t = self.w["ra.weight"].transpose(1, 2).contiguous()
        self._ri_t = self.w["ri.weight"].transpose(1, 2).contiguous()
        self._ra_b = self.w["ra.bias"].to(torch.float32).reshape(-1).contiguous()
        self._ri_b = self.w["ri.bias"].to(torch.float32).reshape(-1).contiguous()
        self._lam = self.w["lam"].to(torch.float32).contiguous()

    def forward(self, x: torch.Tensor, batch, cache) -> torch.Tensor:
        return self.forward_branch(x, batch, cache).value()

    def forward_branch(self, x: torch.Tensor, batch, cache) -> BranchOutput:
        C = self.channels
        state = cache.state
        # the gates and the recurrence are formed from the float32 sums of this product
        proj = self.in_proj.forward(x, out_dtype=torch.float32)
        u = ops.short_conv(proj, C, C, self.w["conv.weight"], self.w["conv.bias"], state.get("conv"), batch.seq_of_token,
                           batch.slot_ids, torch.float32, single_tokens=batch.is_decode)
        a, b = ops.rglru_gates(u, self._ra_t, self._ra_b, self._ri_t, self._ri_b, self._lam, self.decay_constant, batch.seq_of_token)
        mixed = ops.rglru_scan(a, b, proj[:, :C], self.activation, state["S"], batch.seq_starts, batch.seq_of_token, batch.slot_ids,
                               batch.n_seqs, x.dtype, zero_rows=batch.is_decode)
        return BranchOutput(mixed, self.out)


register_part("mixer", "rglru", RecurrentGatedUnit)
