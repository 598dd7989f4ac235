"""Attention whose keys and values are projections of one small latent per token.

Every token leaves two things in the cache: the RMS-normed latent c (kv_rank numbers) and a rotated key part
that all heads share (rot_dim numbers).  Head h's key is [Uk_h c | shared part], its value Uv_h c.  Because
(Uk_h c) . q = c . (Uk_h^T q), the mixer never forms keys or values: it takes each head's query into the latent
space, runs attention as one shared kv head over the cached rows, and takes the result out through Uv_h.  Whole
prompts, portions of prompts and single tokens run the same kernels over the same cache, so how a sequence is cut
into steps changes nothing beyond rounding.

Options, all constructor arguments: queries through a latent of their own with an RMS norm (q_rank; 0: the queries
are one projection of the mixer's input), no rotated part at all (rot_dim 0, attention without positions), a sink logit
per head in the softmax's denominator, a sigmoid gate per head or per output element (read from the mixer's input), a
window, and `owns_kv=False` for a layer that reads the latent and key part that another layer cached (it then has
no down-projection for them; its Uk, Uv, queries and everything else are its own).
"""

from __future__ import annotations

from typing import Optional

import torch

from ..cache import KVNeed
from ..kernels import ops
from .base import BranchOutput, Mixer, register_part
from .linear import Linear
from .position import PositionEncoding


class LatentAttention(Mixer):
    def __init__(
        self,
        width: int,
        nheads: int,
        dim: int,
        rot_dim: int,
        vdim: int,
        q_rank: int,
        kv_rank: int,
        scale: float,
        eps: float = 1e-6,
        sink: bool = False,
        output_gate: bool = False,
        owns_kv: bool = True,
        window: int = 0,
        position_encoder: Optional[PositionEncoding] = None,
    ):
        super().__init__()
        if min(nheads, dim, vdim, kv_rank) <= 0 or q_rank < 0 or rot_dim < 0 or rot_dim % 2:
            raise ValueError("latent attention needs positive sizes and an even rotated size")
        if rot_dim and position_encoder is None:
            raise ValueError("a rotated key part needs a position encoding")
        self.width, self.nheads, self.dim, self.rot_dim, self.vdim = width, nheads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank, self.scale, self.eps = q_rank, kv_rank, float(scale), float(eps)
        if output_gate not in (False, None, True, "head", "element"):
            raise ValueError(f"output_gate {output_gate!r} is not one of False, True, 'head', 'element'")
        self.has_sink, self.has_gate, self.owns_kv, self.window = bool(sink), bool(output_gate), bool(owns_kv), int(window)
        self.gate_cols = 0 if not output_gate else (nheads * vdim if output_gate == "element" else nheads)
        self.position_encoder = position_encoder
        # one product for everything that reads the mixer's input: [query latent (or the queries themselves) | gate logits |
        # kv latent, shared key part]
        self.q_cols = q_rank if q_rank else nheads * (dim + rot_dim)
        self.gate_col = self.q_cols
        self.kv_col = self.q_cols + self.gate_cols
        self.down = self.add_child("down", Linear(width, self.kv_col + ((kv_rank + rot_dim) if owns_kv else 0)))
        if q_rank:
            self.declare("q_norm.weight", (q_rank,), init="ones", kind="scale")
        if owns_kv:
            self.declare("kv_norm.weight", (kv_rank,), init="ones", kind="scale")
        if q_rank:
            self.uq = self.add_child("uq", Linear(q_rank, nheads * (dim + rot_dim)))
        self.declare("uk.weight", (nheads * dim, kv_rank))
        self.declare("uv.weight", (nheads * vdim, kv_rank))
        if sink:
            self.declare("sink", (nheads,), init="zeros", kind="scale")
        self.o = self.add_child("o", Linear(nheads * vdim, width))
        self._uk_t = self._uv = self._sink = None
        self._mfma = False  # decided when the model's type is known (finalize)

    def unfused_parameters(self) -> dict:
        """The fused down-projection as the tensors it is made of, in the order of its rows (what the model's
        state_dict(fused_weights=False) shows in its place)."""
        H = self.nheads
        pieces = [("dq" if self.q_rank else "q", self.q_cols)] + ([("g", self.gate_cols)] if self.has_gate else []) + ([("dkv", self.kv_rank + self.rot_dim)] if self.owns_kv else [])
        return {"down": tuple(pieces)}

    def kv_need(self) -> Optional[KVNeed]:
        """One row [latent | shared key part] per token.  Where the matrix-core kernel runs (bfloat16, sizes that fit
        it) the latent is kept a second time, transposed, as that kernel's values."""
        if self._mfma:
            return KVNeed(1, self.kv_rank + self.rot_dim, self.window, values=True, value_dim=self.kv_rank)
        return KVNeed(1, self.kv_rank + self.rot_dim, self.window, values=False)

    @property
    def graph_safe(self) -> bool:
        return getattr(self.position_encoder, "graph_safe", True)

    def check_step(self, max_position: int) -> None:
        if self.position_encoder is not None:
            self.position_encoder.check_positions(max_position)

    def finalize(self, device, dtype) -> None:
        H, D, R, V = self.nheads, self.dim, self.kv_rank, self.vdim
        self._mfma = dtype == torch.bfloat16 and ops.latent_attention_fits_mfma(R, self.rot_dim) and (H * (R + self.rot_dim)) % 8 == 0
        # Uk_h^T as rows of K = dim contiguous elements: the product that takes a query into the latent space
        self._uk_t = self.w["uk.weight"].view(H, D, R).transpose(1, 2).contiguous()
        self._uv = self.w["uv.weight"].view(H, V, R)
        self._sink = self.w["sink"].to(torch.float32).contiguous() if self.has_sink else None
        if self.position_encoder is not None and self.rot_dim:
            tables = self.position_encoder.rotary_tables()
            if tables is None or tables[2] != self.rot_dim:
                raise ValueError("latent attention rotates by a table of exactly its rotated size")

    def forward(self, x: torch.Tensor, batch, cache) -> torch.Tensor:
        return self.forward_branch(x, batch, cache).value()

    def forward_branch(self, x: torch.Tensor, batch, cache) -> BranchOutput:
        H, D, P, R, V = self.nheads, self.dim, self.rot_dim, self.kv_rank, self.vdim
        T = x.shape[0]
        table = batch.block_tables[cache.group]
        cos = sin = None
        if P:
            cos, sin, _ = self.position_encoder.tables_for_step(batch)
        # norms, gates and everything that enters the cache are formed from the float32 sums of this product
        down = self.down.forward(x, out_dtype=torch.float32)
        if cache.owns:
            if not self.owns_kv:
                raise RuntimeError("this layer has no down-projection for keys and values: it must read another layer's cache")
            ops.latent_kv_write(down, self.kv_col, R, P, self.w["kv_norm.weight"], self.eps, batch.positions, batch.seq_of_token,
                                table, cos, sin, cache.keys, cache.values)
        if self.q_rank:
            cq = ops.rms_norm_cols(down, 0, self.q_rank, self.w["q_norm.weight"], self.eps, x.dtype)
            q = self.uq.forward(cq)
        else:
            q = down[:, : self.q_cols] if down.dtype == x.dtype else ops.cast_cols(down, 0, self.q_cols, x.dtype)
        qa = torch.empty(T, H * (R + P), dtype=x.dtype, device=x.device)
        if P:
            ops.latent_q_rotate(q, qa, H, D, P, R, batch.positions, cos, sin)
        ops.headwise_linear(q, D + P, self._uk_t, qa, R + P)
        mixed_latent = ops.latent_attention(qa, batch.positions, batch.seq_of_token, table, cache.keys, self._sink, H, R, P,
                                            self.scale, self.window, decode=batch.is_decode, max_context=batch.context_bound,
                                            vt_cache=cache.values)
        mixed = torch.empty(T, H * V, dtype=x.dtype, device=x.device)
        gate = down[:, self.gate_col : self.gate_col + self.gate_cols] if self.has_gate else None
        if self.gate_cols == H * V:  # a gate per output element: behind the product that leaves the latent space
            ops.headwise_linear(mixed_latent, R, self._uv, mixed, V)
            mixed = ops.gate_mul(mixed, gate, "sigmoid")
        else:
            ops.headwise_linear(mixed_latent, R, self._uv, mixed, V, gate=gate)
        return BranchOutput(mixed, self.o)


register_part("mixer", "latent_attention", LatentAttention)
