"""Multi-head attention with grouped kv heads over the paged cache: the mixer of Llama.

The reference's order of operations (fms/modules/attention.py:870-937): one fused
projection split into [H*D | K*D | K*D]; rotate queries and keys; append keys and
values to the cache; causal scaled-dot-product attention in which query head h reads
kv head h // (H/K) (:241-250) with scale 1/sqrt(D) unless given (:768-784); output
projection.  Here the rotation and the cache append are one kernel, and attention
reads the cache directly, so a step may bring any number of new tokens per sequence.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from ..cache import KVNeed
from ..kernels import ops
from .base import BranchOutput, Mixer, Part, register_part, split_normed
from .linear import Linear
from .position import PositionEncoding


class LayerCache:
    """What a mixer sees of the cache for one schedule entry."""

    def __init__(self, group: int, keys: Optional[torch.Tensor], values: Optional[torch.Tensor], owns: bool, state: dict):
        self.group, self.keys, self.values, self.owns, self.state = group, keys, values, owns, state


def distance_buckets(rows: int, far: float) -> list:
    """The table row of every distance n = 0, 1, ... up to the first one that falls into the last row (which serves all
    larger distances): n itself below rows/2, then rows/2 + floor(log(n / (rows/2)) / log(far / (rows/2)) * (rows - rows/2)),
    at most rows - 1.  The logarithms are taken in float32, as a model that forms its buckets on tensors does."""
    near = rows // 2
    out = list(range(near))
    n = near
    while True:
        steps = torch.log(torch.tensor(n, dtype=torch.float32) / near) / math.log(far / near) * (rows - near)
        bucket = min(rows - 1, near + int(steps.to(torch.long)))
        out.append(bucket)
        if bucket == rows - 1:
            return out
        n += 1


class MultiHeadAttention(Mixer):
    def __init__(
        self,
        width: int,
        nheads: int,
        kvheads: int,
        head_dim: int,
        use_bias: bool = False,
        position_encoder: Optional[PositionEncoding] = None,
        scale_factor: Optional[float] = None,
        window: int = 0,
        soft_cap: float = 0.0,
        value_dim: Optional[int] = None,
        qkv_bias: Optional[bool] = None,
        out_bias: Optional[bool] = None,
        qk_norm: Optional[str] = None,
        norm_eps: float = 1e-6,
        output_gate=False,
        chunk: int = 0,
        keep_first: int = 0,
        sink: bool = False,
        distance_bias: Optional[dict] = None,
        value_mix: Optional[str] = None,
    ):
        """value_dim: the size of a value (and of an output head) if it is not head_dim.  qkv_bias, out_bias: biases of the
        input and the output projection (default: use_bias for both).  qk_norm "projection": queries and keys pass an RMS
        norm over their whole projection (all heads at once, plain weights, norm_eps), before rotation; "head": over
        every head by itself, with one weight of head_dim entries for all heads.  output_gate (True or "element"): the
        concatenated heads are multiplied by sigmoid(W_g h), h the mixer's input, before the output projection; "head":
        one such gate per head.
        chunk c > 0 (no window then): positions are cut into runs of c from the sequence's start, and a query sees the
        keys of its own run only.  keep_first: with a window, the sequence's first keys that every later query still sees
        (at their true positions).  sink: a learned logit per head in the softmax's denominator, with neither key nor
        value.  distance_bias {"rows": B, "far": D}: a learned table [B, heads] added to the scores by bucketed distance
        n: row n below B/2, then B/2 + floor(log(n / (B/2)) / log(D / (B/2)) * (B - B/2)), at most B - 1.
        value_mix: "first": the step's values are handed to later layers as they are; "blend": the values become
        (1 - lambda) v + lambda v_first with a learned lambda and the values that the "first" layer left for the same
        token (the blended values are what is cached)."""
        super().__init__()
        if kvheads <= 0 or nheads % kvheads:
            raise ValueError(f"{nheads} query heads are no multiple of {kvheads} kv heads")
        if head_dim % 2 or head_dim > 256:
            raise ValueError(f"head size {head_dim} must be even and at most 256")
        self.width, self.nheads, self.kvheads, self.head_dim = width, nheads, kvheads, head_dim
        self.scale = float(scale_factor) if scale_factor is not None else 1.0 / math.sqrt(head_dim)
        self.window = int(window)
        self.soft_cap = float(soft_cap)  # scores become soft_cap * tanh(score / soft_cap); 0: no cap
        if self.soft_cap < 0:
            raise ValueError(f"soft_cap {soft_cap} must be zero (none) or positive")
        self.position_encoder = position_encoder
        self.value_dim = int(value_dim) if value_dim else head_dim
        if not 0 < self.value_dim <= 256:
            raise ValueError(f"value size {self.value_dim} must be at most 256")
        if qk_norm not in (None, "projection", "head"):
            raise ValueError(f"qk_norm {qk_norm!r} is not one of None, 'projection', 'head'")
        if output_gate not in (False, None, True, "element", "head"):
            raise ValueError(f"output_gate {output_gate!r} is not one of False, True, 'element', 'head'")
        self.qk_norm, self.norm_eps, self.output_gate = qk_norm, float(norm_eps), bool(output_gate)
        self.gate_per_head = output_gate == "head"
        self.chunk, self.keep_first, self.has_sink = int(chunk), int(keep_first), bool(sink)
        if self.chunk < 0 or self.keep_first < 0 or (self.chunk and (self.window or self.keep_first)):
            raise ValueError("chunks go with neither a window nor kept first keys, and no size is negative")
        if self.keep_first and not self.window:
            self.keep_first = 0  # without a window every key stays visible anyway
        self.distance_bias = dict(distance_bias) if distance_bias else None
        if self.distance_bias is not None and not (self.distance_bias["rows"] >= 2 and self.distance_bias["far"] > self.distance_bias["rows"] // 2):
            raise ValueError("a distance table needs at least two rows and a far distance beyond half of them")
        if value_mix not in (None, "first", "blend"):
            raise ValueError(f"value_mix {value_mix!r} is not one of None, 'first', 'blend'")
        if value_mix and not qk_norm:
            raise NotImplementedError("values are handed on and blended by the kernel that norms queries and keys")
        self.value_mix = value_mix
        qkv_bias = use_bias if qkv_bias is None else bool(qkv_bias)
        out_bias = use_bias if out_bias is None else bool(out_bias)
        # the steps beyond Llama's attention run a path of their own; without them nothing changes
        self.extended = bool(self.qk_norm or self.output_gate or self.value_dim != head_dim or self.value_mix)
        self.n_q, self.n_k, self.n_v = nheads * head_dim, kvheads * head_dim, kvheads * self.value_dim
        in_proj = self.add_child("in_proj", Part())
        # with an output gate the gate's rows follow the values: everything that reads the mixer's input is one product
        self.n_gate = (nheads if self.gate_per_head else nheads * self.value_dim) if self.output_gate else 0
        rows = self.n_q + self.n_k + self.n_v + self.n_gate
        self.qkv = in_proj.add_child("qkv_fused", Linear(width, rows, qkv_bias))
        if self.qk_norm:
            self.declare("q_norm.weight", (head_dim if qk_norm == "head" else self.n_q,), init="ones", kind="scale")
            self.declare("k_norm.weight", (head_dim if qk_norm == "head" else self.n_k,), init="ones", kind="scale")
        if self.has_sink:
            self.declare("sink", (nheads,), init="zeros", kind="scale")
        if self.distance_bias is not None:
            self.declare("rel", (self.distance_bias["rows"], nheads), init="normal", kind="scale")
        if self.value_mix:
            self.declare("vmix", (), init="zeros", kind="scale")  # the "first" layer has one too, and does not use it
        self._sink = self._bias_by_distance = self._lambda = None
        self.dense = self.add_child("dense", Linear(nheads * self.value_dim, width, out_bias))

    def unfused_parameters(self) -> dict:
        """The fused projection as the parts it is made of: fused local name -> ((local name, rows), ...), in the
        order of the rows (fms/modules/attention.py:666-687)."""
        pieces = (("in_proj.query", self.n_q), ("in_proj.key", self.n_k), ("in_proj.value", self.n_v))
        if self.output_gate:
            pieces += (("in_proj.gate", self.n_gate),)
        return {"in_proj.qkv_fused": pieces}

    def output_projection(self) -> Linear:
        return self.dense

    # ---- what the mixer asks of the cache ---------------------------------
    def kv_need(self) -> Optional[KVNeed]:
        value_dim = self.value_dim if self.value_dim != self.head_dim else 0
        return KVNeed(self.kvheads, self.head_dim, self.window, value_dim=value_dim, keep_first=self.keep_first, chunk=self.chunk)

    def finalize(self, device, dtype) -> None:
        """What the kernels read in float32: the sink logits, the blending factor, and the distance table laid out by
        distance (row n of every head for n up to the first distance of the last bucket, which serves all beyond)."""
        if self.has_sink:
            self._sink = self.w["sink"].to(torch.float32).contiguous()
        if self.value_mix == "blend":
            self._lambda = self.w["vmix"].to(torch.float32).reshape(1).contiguous()
        if self.distance_bias is not None:
            rows, far = self.distance_bias["rows"], float(self.distance_bias["far"])
            buckets = distance_buckets(rows, far)
            table = self.w["rel"].to(torch.float32)  # [rows, heads]
            self._bias_by_distance = table[torch.tensor(buckets, device=table.device)].t().contiguous()  # [heads, L]

    def state_need(self):
        return None

    @property
    def graph_safe(self) -> bool:
        return getattr(self.position_encoder, "graph_safe", True)

    def check_step(self, max_position: int) -> None:
        if self.position_encoder is not None:
            self.position_encoder.check_positions(max_position)

    def _score_slopes(self) -> Optional[torch.Tensor]:
        return self.position_encoder.score_slopes(self.nheads) if self.position_encoder is not None else None

    def prefill_qblock(self, n_tokens: int, dtype) -> int:
        if (dtype != torch.bfloat16 or self.head_dim % 16 or self._score_slopes() is not None or self.value_dim != self.head_dim
                or ((self.keep_first or self.distance_bias is not None) and ops.prefill_extras_are_generic(self.head_dim))
                or ops.prefill_cap_is_generic(self.head_dim, self.soft_cap)):
            return 0  # the generic kernel takes tokens one by one
        return ops.prefill_qblock(self.nheads, self.kvheads, self.head_dim, n_tokens)

    def _fused_decode(self, rows: int, dtype, batch) -> bool:
        """True if projection, rotation and cache write of this step run as one kernel."""
        rotates_by_table = self.position_encoder is None or self.position_encoder.rotary_tables() is not None
        return (not self.extended and batch.is_decode and rows <= ops.QKV_ROPE_MAX_ROWS and dtype == torch.bfloat16
                and self.qkv.w["weight"].dtype == torch.bfloat16 and self.head_dim % 16 == 0 and self.width % 8 == 0
                and rotates_by_table)

    def accepts_normed_rows(self, rows: int, dtype, batch) -> bool:
        return self._fused_decode(rows, dtype, batch)

    def forward(self, x: torch.Tensor, batch, cache: LayerCache) -> torch.Tensor:
        return self.forward_branch(x, batch, cache).value()

    def forward_branch(self, x, batch, cache: LayerCache, out: Optional[torch.Tensor] = None, out_scale: float = 1.0) -> BranchOutput:
        """out (rows [T, heads * value size] of any stride) and out_scale: where the input of the output projection is
        written, and a factor on it, for a caller that runs this mixer beside another and projects both at once."""
        x, row_norm = split_normed(x)
        H, K, D = self.nheads, self.kvheads, self.head_dim
        table = batch.block_tables[cache.group]
        tables = self.position_encoder.tables_for_step(batch) if self.position_encoder is not None else None
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        keys, values = (cache.keys, cache.values) if cache.owns else (None, None)
        weight = self.qkv.w["weight"]
        gate = None
        if self.extended:
            if row_norm is not None:
                raise RuntimeError("a deferred norm reached a step that does not take one")
            # norms and the gate are formed from the float32 sums of the projection
            proj = self.qkv.forward(x, out_dtype=torch.float32)
            if self.qk_norm:
                v_first = None
                if self.value_mix == "blend":
                    v_first = batch.shared.get("first_values")
                    if v_first is None or v_first.shape[1] != self.n_v:
                        raise RuntimeError("values are blended with those of an earlier layer of the step, and none has left values of this size")
                qkv = ops.qk_projection_norm(proj, self.n_q, self.n_k, self.n_v, self.w["q_norm.weight"], self.w["k_norm.weight"],
                                             self.norm_eps, x.dtype, batch.seq_of_token, norm_dim=D if self.qk_norm == "head" else 0,
                                             v_first=v_first, v_lambda=self._lambda if v_first is not None else None)
                if self.value_mix == "first":
                    batch.shared["first_values"] = qkv[:, self.n_q + self.n_k :]
            else:
                qkv = ops.cast_cols(proj, 0, self.n_q + self.n_k + self.n_v, x.dtype)
            if self.output_gate:
                gate = proj[:, self.n_q + self.n_k + self.n_v :]
            if tables is None and self.position_encoder is not None:
                self.position_encoder.adjust_qk(qkv, batch, H, K, D)
            ops.rope_kv_write(qkv, batch.positions, batch.seq_of_token, table, cos, sin, rot, keys, values, H, K, D, self.value_dim)
        elif self._fused_decode(x.shape[0], x.dtype, batch):
            # decode: projection, rotation and cache write in one kernel
            qkv = ops.qkv_rope_write(x, weight, self.qkv.w.get("bias"), batch.positions, batch.seq_of_token, table,
                                     cos, sin, rot, keys, values, H, K, D, row_norm=row_norm)
        else:
            if row_norm is not None:
                raise RuntimeError("a deferred norm reached a step that does not take one")
            qkv = self.qkv.forward(x)
            if tables is None and self.position_encoder is not None:
                self.position_encoder.adjust_qk(qkv, batch, H, K, D)
            ops.rope_kv_write(qkv, batch.positions, batch.seq_of_token, table, cos, sin, rot, keys, values, H, K, D)
        size = 0 if batch.is_decode else self.prefill_qblock(batch.n_tokens, x.dtype)
        qb_start, qb_len = batch.qblocks.get(size, (None, None))
        mixed = ops.attention(
            qkv, batch.positions, batch.seq_of_token, table, cache.keys, cache.values, H, K, D, self.scale, self.window,
            decode=batch.is_decode, max_context=batch.context_bound,
            qblock_start=qb_start, qblock_len=qb_len, qblock_tokens=size,
            row_order=batch.rows_by_length if batch.is_decode else None,
            score_slopes=self._score_slopes(), soft_cap=self.soft_cap, value_dim=self.value_dim,
            chunk=self.chunk, keep_first=self.keep_first, sink=self._sink, distance_bias=self._bias_by_distance,
        )
        if gate is not None or out is not None or out_scale != 1.0:
            mixed = ops.gate_mul(mixed, gate, "sigmoid", out_scale, out=out, group=self.value_dim if self.gate_per_head else 1)
        return BranchOutput(mixed, self.dense)


register_part("mixer", "attention", MultiHeadAttention)
