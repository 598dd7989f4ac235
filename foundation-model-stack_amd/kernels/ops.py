"""The kernels as functions of torch tensors.

torch tensors are used as device buffers only; every computation below is a
HIP kernel of this package, with one exception that is named where it happens
(large bfloat16 matrix products go to the vendor library through
``torch.matmul``, as the reference's linear layers do).  Each wrapper checks on
the host what its kernel and grid assume before launching.
"""

from __future__ import annotations

import ctypes
import math
from typing import Optional

import torch

from .library import check, load

F32, BF16 = 0, 1
# the names of the reference (fms/utils/activation.py:14-24) and "identity"; the numbers are FMS_ACT_* of csrc/fmsamd.h
ACTIVATIONS = {"silu": 0, "swish": 0, "gelu": 1, "relu": 2, "identity": 3, "sigmoid": 4, "tanh": 5, "mish": 6,
               "gelu-tanh": 7, "gelu_pytorch_tanh": 7}
PAGE_TOKENS = 64


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    raise TypeError(f"fms_amd kernels take float32 and bfloat16, not {dtype}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("fms_amd kernels run on the GPU only; got a CPU tensor (there is no CPU fallback)")


def _need_i32(name: str, t: torch.Tensor) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{name} must be a contiguous int32 tensor")


def _rows2d(name: str, t: torch.Tensor) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with a contiguous last dimension, got shape {tuple(t.shape)} strides {t.stride()}")


# --------------------------------------------------------------------------
def embed(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 rows of `table` for int32 `ids` [T], times `scale` -> [T, width]."""
    _need_cuda(ids, table)
    _need_i32("ids", ids)
    if table.dim() != 2 or not table.is_contiguous():
        raise ValueError("embedding table must be a contiguous [vocab, width] tensor")
    out = torch.empty(ids.numel(), table.shape[1], dtype=torch.float32, device=table.device)
    check(load().fmsamd_embed(ids.data_ptr(), table.data_ptr(), _code(table.dtype), out.data_ptr(), ids.numel(),
                              table.shape[1], table.shape[0], float(scale), _stream()))
    return out


def add_norm(
    resid: torch.Tensor,
    branch: Optional[torch.Tensor],
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
    use_mean: bool = False,
) -> torch.Tensor:
    """resid += branch (in place, float32); returns norm(resid) * weight + bias in `out_dtype`.

    With `rows` (int32 indices) only those rows are produced and resid is left as it is.
    """
    _need_cuda(resid, branch, weight, bias, rows)
    if resid.dtype != torch.float32 or resid.dim() != 2 or not resid.is_contiguous():
        raise ValueError("the residual stream must be a contiguous float32 [T, width] tensor")
    T, width = resid.shape
    if branch is not None:
        if branch.shape != resid.shape or not branch.is_contiguous() or branch.dtype != out_dtype:
            raise ValueError(f"branch must be contiguous {tuple(resid.shape)} of {out_dtype}, got {tuple(branch.shape)} {branch.dtype}")
    wdtype = out_dtype
    for name, t in (("weight", weight), ("bias", bias)):
        if t is not None:
            if t.shape != (width,) or not t.is_contiguous():
                raise ValueError(f"norm {name} must be a contiguous [{width}] tensor, got {tuple(t.shape)}")
            wdtype = t.dtype
    if weight is not None and bias is not None and weight.dtype != bias.dtype:
        raise TypeError("norm weight and bias must have one dtype")
    n_out = T
    if rows is not None:
        _need_i32("rows", rows)
        n_out = rows.numel()
    out = torch.empty(n_out, width, dtype=out_dtype, device=resid.device)
    check(load().fmsamd_add_norm(resid.data_ptr(), _ptr(branch), _code(out_dtype), _ptr(weight), _ptr(bias), _code(wdtype),
                                 out.data_ptr(), _ptr(rows), n_out, width, float(eps), int(use_mean), _stream()))
    return out


def gated_act(gu: torch.Tensor, bias: Optional[torch.Tensor], activation: str) -> torch.Tensor:
    """[T, 2*hidden] (gate first) -> act(gate + b) * (up + b) [T, hidden]."""
    _need_cuda(gu, bias)
    if gu.dim() != 2 or not gu.is_contiguous() or gu.shape[1] % 2:
        raise ValueError("gated_act takes a contiguous [T, 2*hidden] tensor")
    T, hidden = gu.shape[0], gu.shape[1] // 2
    if bias is not None and (bias.shape != (2 * hidden,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{2 * hidden}] tensor")
    out = torch.empty(T, hidden, dtype=gu.dtype, device=gu.device)
    for t0 in range(0, T, 65535):
        n = min(65535, T - t0)
        check(load().fmsamd_gated_act(gu[t0:].data_ptr(), _ptr(bias), _code(bias.dtype) if bias is not None else 0,
                                      out[t0:].data_ptr(), _code(gu.dtype), n, hidden, ACTIVATIONS[activation], _stream()))
    return out


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _need_cuda(x)
    if x.dtype == dtype:
        return x
    if not x.is_contiguous():
        raise ValueError("cast takes a contiguous tensor")
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    check(load().fmsamd_cast(x.data_ptr(), _code(x.dtype), out.data_ptr(), _code(dtype), x.numel(), _stream()))
    return out


def advance_positions_(positions: torch.Tensor, seq_of_token: torch.Tensor) -> None:
    """positions += 1 on the live rows (seq_of_token >= 0) of a fixed-size decode batch."""
    _need_cuda(positions, seq_of_token)
    _need_i32("positions", positions)
    _need_i32("seq_of_token", seq_of_token)
    if positions.numel() != seq_of_token.numel():
        raise ValueError("positions and seq_of_token must have one entry per row")
    check(load().fmsamd_advance_positions(positions.data_ptr(), seq_of_token.data_ptr(), positions.numel(), _stream()))


def bias_add_(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    _need_cuda(x, bias)
    if x.dim() != 2 or not x.is_contiguous() or bias.shape != (x.shape[1],) or not bias.is_contiguous():
        raise ValueError("bias_add_ takes a contiguous [rows, cols] tensor and a [cols] bias")
    check(load().fmsamd_bias_add(x.data_ptr(), _code(x.dtype), bias.data_ptr(), _code(bias.dtype), x.shape[0], x.shape[1], _stream()))
    return x


# --------------------------------------------------------------------------
def rope_table(freqs: torch.Tensor, max_pos: int):
    """cos and sin of position * freqs, float32 [max_pos, len(freqs)]."""
    _need_cuda(freqs)
    if freqs.dtype != torch.float32 or freqs.dim() != 1 or not freqs.is_contiguous():
        raise ValueError("freqs must be a contiguous float32 vector")
    half = freqs.numel()
    cos = torch.empty(max_pos, half, dtype=torch.float32, device=freqs.device)
    sin = torch.empty_like(cos)
    check(load().fmsamd_rope_table(freqs.data_ptr(), cos.data_ptr(), sin.data_ptr(), max_pos, half, _stream()))
    return cos, sin


def _check_cache(k_cache: torch.Tensor, v_cache: torch.Tensor, kvheads: int, head_dim: int, dtype: torch.dtype,
                 value_dim: int = 0) -> int:
    shape = (kvheads, PAGE_TOKENS, head_dim)
    if k_cache.dim() != 4 or tuple(k_cache.shape[1:]) != shape or not k_cache.is_contiguous():
        raise ValueError(f"key cache must be contiguous [pages, {kvheads}, {PAGE_TOKENS}, {head_dim}], got {tuple(k_cache.shape)}")
    vshape = (kvheads, value_dim or head_dim, PAGE_TOKENS)
    if v_cache.dim() != 4 or tuple(v_cache.shape[1:]) != vshape or not v_cache.is_contiguous():
        raise ValueError(f"value cache must be contiguous [pages, {kvheads}, {value_dim or head_dim}, {PAGE_TOKENS}], got {tuple(v_cache.shape)}")
    if k_cache.dtype != dtype or v_cache.dtype != dtype or k_cache.shape[0] != v_cache.shape[0]:
        raise TypeError("key and value cache must have the dtype of the queries and equal page counts")
    return k_cache.shape[0]


def _check_batch_index(positions, seq_of_token, block_table, n_tokens: int) -> None:
    _need_i32("positions", positions)
    _need_i32("seq_of_token", seq_of_token)
    if block_table.dtype != torch.int32 or block_table.dim() != 2 or block_table.stride(1) != 1:
        raise TypeError("block_table must be an int32 [sequences, pages] tensor")
    if positions.numel() < n_tokens or seq_of_token.numel() < n_tokens:
        raise ValueError("positions and seq_of_token must have an entry per token")


class RowNorm:
    """A row norm left to the product that reads the rows.  The rows hold stream * norm weight; `partials`
    [M, count] float32 are partial sums of squares of the stream's rows; the product multiplies its result
    by rsqrt(sum / K + eps) per row before the bias."""

    def __init__(self, partials: torch.Tensor, eps: float):
        if partials.dtype != torch.float32 or partials.dim() != 2 or not partials.is_contiguous():
            raise ValueError("the partial sums of a deferred row norm are a contiguous float32 [M, count] tensor")
        self.partials, self.eps = partials, float(eps)


def _skinny_workspace(rows: int, weight_rows: int, K: int, device):
    """(pointer, bytes) of the workspace a product for `rows` rows of x needs; (None, 0) up to 16 rows."""
    n = load().fmsamd_gemm_skinny_workspace(rows, weight_rows, K)
    if n <= 0:
        return None, 0
    ws = torch.empty(n // 4, dtype=torch.float32, device=device)
    return ws, n


class _RowScaleArg(ctypes.Structure):
    _fields_ = [("partials", ctypes.c_void_p), ("count", ctypes.c_int), ("eps", ctypes.c_float)]


def _row_scale(row_norm: Optional[RowNorm], rows: int):
    if row_norm is None:
        return None
    _need_cuda(row_norm.partials)
    if row_norm.partials.shape[0] != rows:
        raise ValueError(f"deferred row norm has {row_norm.partials.shape[0]} rows, the product {rows}")
    return ctypes.byref(_RowScaleArg(row_norm.partials.data_ptr(), row_norm.partials.shape[1], row_norm.eps))


def qkv_rope_write(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    positions: torch.Tensor,
    seq_of_token: torch.Tensor,
    block_table: torch.Tensor,
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    rot_dim: int,
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    nheads: int,
    kvheads: int,
    head_dim: int,
    row_norm: Optional[RowNorm] = None,
) -> torch.Tensor:
    """The fused qkv projection of a decode step (at most QKV_ROPE_MAX_ROWS rows, bfloat16): x W^T (+ bias), q and k
    rotated, k and v written into their cache pages.  Returns the [M, (H+2K)*D] buffer whose query
    columns hold the rotated queries (its other columns are not written).  Equal to `linear` followed
    by `rope_kv_write`."""
    _need_cuda(x, weight, bias, positions, seq_of_token, block_table, cos, sin, k_cache, v_cache)
    _rows2d("x", x)
    M, K = x.shape
    N = (nheads + 2 * kvheads) * head_dim
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or tuple(weight.shape) != (N, K) or not weight.is_contiguous():
        raise ValueError(f"qkv_rope_write takes bfloat16 x [M, {K}] and a contiguous bfloat16 weight [{N}, {K}]")
    if M > QKV_ROPE_MAX_ROWS or K % 8 or x.stride(0) % 8 or N % 16:
        raise ValueError(f"qkv_rope_write: at most {QKV_ROPE_MAX_ROWS} rows, K a multiple of 8, the output row a multiple of 16")
    if bias is not None and (bias.shape != (N,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{N}] tensor")
    _check_batch_index(positions, seq_of_token, block_table, M)
    max_pos = 0
    if cos is not None:
        if cos.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim:
            raise ValueError("cos/sin tables must be float32 [max_pos, rot_dim/2]")
        if not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("cos/sin tables must be contiguous")
        max_pos = cos.shape[0]
    if k_cache is not None:
        _check_cache(k_cache, v_cache, kvheads, head_dim, torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    ws, ws_bytes = _skinny_workspace(M, N, K, x.device)
    check(load().fmsamd_qkv_rope_skinny_bf16(
        x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), _code(bias.dtype) if bias is not None else 0,
        out.data_ptr(), out.stride(0), M, K, positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
        block_table.stride(0), _ptr(cos), _ptr(sin), rot_dim if cos is not None else 0, max_pos, _ptr(k_cache),
        _ptr(v_cache), nheads, kvheads, head_dim, _row_scale(row_norm, M), _ptr(ws), ws_bytes, _stream()))
    return out


QKV_ROPE_MAX_ROWS = 192


def rope_kv_write(
    qkv: torch.Tensor,
    positions: torch.Tensor,
    seq_of_token: torch.Tensor,
    block_table: torch.Tensor,
    cos: Optional[torch.Tensor],
    sin: Optional[torch.Tensor],
    rot_dim: int,
    k_cache: Optional[torch.Tensor],
    v_cache: Optional[torch.Tensor],
    nheads: int,
    kvheads: int,
    head_dim: int,
    value_dim: int = 0,
) -> None:
    """Rotate q (in place, inside qkv) and k; write k and v of every token into its cache page.
    value_dim (0: head_dim): values of a size of their own; the rows are then [H*D | K*D | K*value_dim].

    The caller guarantees (and the engine checks on the host) that every position is below the
    table length and that block_table holds a valid page for every (sequence, position // 64).
    """
    _need_cuda(qkv, positions, seq_of_token, block_table, cos, sin, k_cache, v_cache)
    _rows2d("qkv", qkv)
    T = qkv.shape[0]
    value_dim = 0 if value_dim == head_dim else int(value_dim)
    if qkv.shape[1] != (nheads + kvheads) * head_dim + kvheads * (value_dim or head_dim):
        raise ValueError(f"qkv has {qkv.shape[1]} columns, expected {(nheads + kvheads) * head_dim + kvheads * (value_dim or head_dim)}")
    _check_batch_index(positions, seq_of_token, block_table, T)
    max_pos = 0
    if cos is not None:
        if cos.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] * 2 != rot_dim:
            raise ValueError("cos/sin tables must be float32 [max_pos, rot_dim/2]")
        if not (cos.is_contiguous() and sin.is_contiguous()):
            raise ValueError("cos/sin tables must be contiguous")
        max_pos = cos.shape[0]
    if k_cache is not None:
        _check_cache(k_cache, v_cache, kvheads, head_dim, qkv.dtype, value_dim)
    check(load().fmsamd_rope_kv_write(qkv.data_ptr(), _code(qkv.dtype), qkv.stride(0), positions.data_ptr(),
                                      seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0),
                                      _ptr(cos), _ptr(sin), rot_dim if cos is not None else 0, max_pos, _ptr(k_cache),
                                      _ptr(v_cache), T, nheads, kvheads, head_dim, value_dim, _stream()))


def attention(
    q: torch.Tensor,
    positions: torch.Tensor,
    seq_of_token: torch.Tensor,
    block_table: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    nheads: int,
    kvheads: int,
    head_dim: int,
    scale: float,
    window: int = 0,
    *,
    decode: bool = False,
    max_context: int = 0,
    qblock_start: Optional[torch.Tensor] = None,
    qblock_len: Optional[torch.Tensor] = None,
    qblock_tokens: int = 0,
    pages_per_block: int = 0,
    waves: int = 0,
    force_generic: bool = False,
    staged: Optional[bool] = None,
    row_order: Optional[torch.Tensor] = None,
    score_slopes: Optional[torch.Tensor] = None,
    soft_cap: float = 0.0,
    value_dim: int = 0,
    chunk: int = 0,
    keep_first: int = 0,
    sink: Optional[torch.Tensor] = None,
    distance_bias: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Causal attention of every token over the cache of its sequence -> [T, nheads*head_dim] (with value_dim, values
    and output heads of that size, through the generic kernel).

    Which keys a query sees beside the causal rule: the last `window` (0: all), of which the sequence's first `keep_first`
    keys are exempt; or, with chunk > 0 (and no window), the keys of the query's own run of `chunk` positions, counted from
    the sequence's start.  sink: float32 [nheads], a logit per head that joins the softmax's denominator and has neither
    key nor value.  distance_bias: float32 [nheads, L], added to the score by distance, min(distance, L - 1), neither
    scaled nor capped.  The matrix-core kernels carry chunks and the sink; kept first keys and the distance bias the
    matrix-core decode kernel, and the matrix-core prompt kernel for head sizes up to 64 and for 128.

    Further terms of the scores (a position encoding that acts on the scores, a capped attention): score_slopes,
    float32 [nheads], adds slope[head] * (key position - query position); soft_cap c > 0 turns a score s into
    c * tanh(s / c) first.  With slopes both types run the generic kernel (the MFMA kernels have no such term); the
    cap they have.

    q is a [T, >= nheads*head_dim] view (the query columns of the qkv rows).  float32 runs the
    generic kernel; bfloat16 runs the MFMA kernels (prefill needs the query blocks, decode the
    largest context).  row_order (decode, optional): int32 [T], the token rows in the order in which the
    kernel's blocks are to take them, longest context first; the result does not depend on it.
    """
    _need_cuda(q, positions, seq_of_token, block_table, k_cache, v_cache)
    _rows2d("q", q)
    T = q.shape[0]
    _check_batch_index(positions, seq_of_token, block_table, T)
    value_dim = 0 if value_dim == head_dim else int(value_dim)
    _check_cache(k_cache, v_cache, kvheads, head_dim, q.dtype, value_dim)
    out = torch.empty(T, nheads * (value_dim or head_dim), dtype=q.dtype, device=q.device)
    lib = load()
    common_tail = (T, nheads, kvheads, head_dim, float(scale), int(window), _stream())
    if score_slopes is not None:
        _need_cuda(score_slopes)
        if score_slopes.dtype != torch.float32 or tuple(score_slopes.shape) != (nheads,) or not score_slopes.is_contiguous():
            raise ValueError(f"score_slopes must be a contiguous float32 [{nheads}] tensor")
    if not (soft_cap >= 0.0 and math.isfinite(soft_cap)):
        raise ValueError(f"soft_cap {soft_cap} must be zero (none) or positive")
    chunk, keep_first = int(chunk), int(keep_first)
    if chunk < 0 or keep_first < 0 or (chunk > 0 and (window > 0 or keep_first > 0)):
        raise ValueError(f"chunks ({chunk}) go with neither a window ({window}) nor kept first keys ({keep_first}), and none is negative")
    if sink is not None:
        _need_cuda(sink)
        if sink.dtype != torch.float32 or tuple(sink.shape) != (nheads,) or not sink.is_contiguous():
            raise ValueError(f"sink must be a contiguous float32 [{nheads}] tensor")
    dist_len = 0
    if distance_bias is not None:
        _need_cuda(distance_bias)
        if distance_bias.dtype != torch.float32 or distance_bias.dim() != 2 or distance_bias.shape[0] != nheads or not distance_bias.is_contiguous():
            raise ValueError(f"distance_bias must be a contiguous float32 [{nheads}, L] tensor")
        dist_len = distance_bias.shape[1]
    prefill_extras = bool(keep_first) or distance_bias is not None  # kept keys or a table: not every matrix-core kernel has them
    if (q.dtype == torch.float32 or force_generic or head_dim % 16 or score_slopes is not None or value_dim
            or (prefill_extras and not decode and (prefill_extras_are_generic(head_dim) or qblock_start is None))
            or (not decode and prefill_cap_is_generic(head_dim, soft_cap))):
        for t0 in range(0, T, 65535):
            n = min(65535, T - t0)
            check(lib.fmsamd_attn_generic(q[t0:].data_ptr(), q.stride(0), out[t0:].data_ptr(), out.stride(0), _code(q.dtype),
                                          positions[t0:].data_ptr(), seq_of_token[t0:].data_ptr(), block_table.data_ptr(),
                                          block_table.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), n, *common_tail[1:-1],
                                          _ptr(score_slopes), float(soft_cap), value_dim, chunk, keep_first, _ptr(sink),
                                          _ptr(distance_bias), dist_len, common_tail[-1]))
        return out
    if decode:
        if max_context <= 0:
            raise ValueError("decode attention needs max_context (an upper bound of every context length)")
        # a window or a chunk bounds the pages a query can see whatever its context: the step is cut for that many, so
        # that long contexts do not launch splits that find no key
        seen = 0
        if window > 0:
            seen = -(-int(window) // PAGE_TOKENS) + 1 + -(-keep_first // PAGE_TOKENS)
        elif chunk > 0:
            seen = -(-chunk // PAGE_TOKENS) + 1
        if seen:
            max_context = min(int(max_context), seen * PAGE_TOKENS)
        n_pages = -(-max_context // PAGE_TOKENS)
        auto_pages, auto_waves = decode_split(T * kvheads, n_pages)
        if pages_per_block <= 0:
            pages_per_block = auto_pages
        if waves <= 0:
            waves = min(auto_waves, pages_per_block)
        n_splits = -(-n_pages // pages_per_block)
        if row_order is not None:
            _need_cuda(row_order)
            _need_i32("row_order", row_order)
            if row_order.numel() != T or not row_order.is_contiguous():
                raise ValueError(f"row_order has {row_order.numel()} entries for {T} tokens")
        ws_bytes = lib.fmsamd_attn_decode_workspace(T, nheads, head_dim, n_splits)
        ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=q.device) if ws_bytes else None
        check(lib.fmsamd_attn_decode_bf16(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), _ptr(ws), ws_bytes,
                                          positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(),
                                          block_table.stride(0), k_cache.data_ptr(), v_cache.data_ptr(), T, nheads, kvheads,
                                          head_dim, float(scale), int(window), int(max_context), int(pages_per_block), int(waves),
                                          int(bool(staged)) if staged is not None else int(head_dim == 128 and not prefill_extras), _ptr(row_order),
                                          float(soft_cap), chunk, _ptr(sink), keep_first, _ptr(distance_bias), dist_len, _stream()))
        return out
    if qblock_start is None or qblock_len is None:
        raise ValueError("bfloat16 prefill attention needs the query blocks of the batch")
    _need_i32("qblock_start", qblock_start)
    _need_i32("qblock_len", qblock_len)
    check(lib.fmsamd_attn_prefill_bf16(q.data_ptr(), q.stride(0), out.data_ptr(), out.stride(0), positions.data_ptr(),
                                       seq_of_token.data_ptr(), qblock_start.data_ptr(), qblock_len.data_ptr(),
                                       qblock_start.numel(), int(qblock_tokens), block_table.data_ptr(), block_table.stride(0),
                                       k_cache.data_ptr(), v_cache.data_ptr(), *common_tail[:-1], float(soft_cap), chunk, _ptr(sink),
                                       keep_first, _ptr(distance_bias), dist_len, common_tail[-1]))
    return out


def decode_split(rows: int, n_pages: int):
    """(pages per split, waves per block) of the decode attention kernel.

    rows = tokens x kv heads.  A compute unit pulls only a small share of the memory bandwidth, so
    the cache has to be spread over all of them: the context bound is cut into as many splits as give
    a few hundred blocks, and at least so many that a block has no more than 128 pages (every sequence
    deals its own pages out evenly over the splits; the waves of a block run their pages as a pipeline,
    so a block of many pages is cheaper than many blocks).  The waves of a block share its pages and merge in LDS, the blocks of a row
    merge in a second kernel."""
    by_rows = min(-(-256 // max(rows, 1)), max(1, n_pages // 8))  # but no splits of under 8 pages: one for each wave
    splits = max(1, min(max(by_rows, -(-n_pages // 128)), n_pages))
    pages = -(-n_pages // splits)
    waves = max(1, min(8 if rows * splits <= 512 else 4, pages))
    return pages, waves


def prefill_cap_is_generic(head_dim: int, soft_cap: float) -> bool:
    """True if capped scores of this head size run the generic kernel in multi-token steps: the matrix-core prefill
    kernel for head sizes between 64 and 128 has no cap."""
    return soft_cap > 0.0 and 64 < head_dim < 128


def prefill_extras_are_generic(head_dim: int) -> bool:
    """True if kept first keys and a distance table of this head size run the generic kernel in multi-token steps: the
    matrix-core prefill kernels carry them for head sizes up to 64 and for 128."""
    return head_dim > 64 and head_dim != 128


def prefill_qblock(nheads: int, kvheads: int, head_dim: int, n_tokens: int) -> int:
    """The number of consecutive query tokens of one sequence that a block of the bfloat16 prefill
    kernel takes, for a step of n_tokens tokens; the step's query blocks are built with it."""
    return load().fmsamd_attn_prefill_qblock(nheads, kvheads, head_dim, n_tokens)


# --------------------------------------------------------------------------
# matrix products
# --------------------------------------------------------------------------
SKINNY_MAX_ROWS = 192
# Up to this many rows the skinny kernel, with the norms, rotation and activation fused into it, beats the
# vendor library followed by those as kernels of their own.
SKINNY_FAST_ROWS = 192


def linear(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    out_dtype: Optional[torch.dtype] = None,
    allow_library: bool = True,
    row_norm: Optional[RowNorm] = None,
) -> torch.Tensor:
    """x [M, K] @ weight[N, K]^T (+ bias) -> [M, N].

    float32 x float32: the FMA kernel (true 32-bit).  bfloat16 x bfloat16: the weight-streaming
    skinny kernels up to 192 rows; above that the vendor library (hipBLASLt through torch.matmul,
    as the reference's nn.Linear does; for float32 output with the float32 sums as they are), or this
    package's MFMA kernel when allow_library is False.
    A float32 weight with bfloat16 activations (a tensor the checkpoint keeps in 32-bit) runs the
    float32 kernel on up-cast activations.
    """
    _need_cuda(x, weight, bias)
    _rows2d("x", x)
    if weight.dim() != 2 or not weight.is_contiguous():
        raise ValueError("weight must be a contiguous [N, K] tensor")
    M, K = x.shape
    N = weight.shape[0]
    if weight.shape[1] != K:
        raise ValueError(f"x has {K} columns, weight has {weight.shape[1]}")
    if bias is not None and (bias.shape != (N,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{N}] tensor")
    out_dtype = out_dtype or x.dtype
    lib = load()
    if row_norm is not None and not (weight.dtype == x.dtype == torch.bfloat16 and M <= SKINNY_FAST_ROWS):
        raise ValueError(f"a deferred row norm goes with the bfloat16 product of at most {SKINNY_FAST_ROWS} rows")
    if weight.dtype == torch.float32:
        xf = x if x.dtype == torch.float32 else cast(x.contiguous(), torch.float32)
        bf = bias if bias is None or bias.dtype == torch.float32 else cast(bias, torch.float32)
        out = torch.empty(M, N, dtype=torch.float32, device=x.device)
        for m0 in range(0, M, 65535 * 64):
            m = min(65535 * 64, M - m0)
            check(lib.fmsamd_gemm_f32(xf[m0:].data_ptr(), xf.stride(0), weight.data_ptr(), _ptr(bf), out[m0:].data_ptr(),
                                      out.stride(0), m, N, K, _stream()))
        return out if out_dtype == torch.float32 else cast(out, out_dtype)
    if weight.dtype != torch.bfloat16:
        raise TypeError(f"weights are float32 or bfloat16, not {weight.dtype}")
    if x.dtype != torch.bfloat16:
        raise TypeError("a bfloat16 weight takes bfloat16 activations")
    bcode = _code(bias.dtype) if bias is not None else 0
    if K % 8 or x.stride(0) % 8:
        # rows that are not 16-byte aligned: the element-wise kernel, so that no width is refused
        if row_norm is not None:
            raise ValueError("a deferred row norm goes with K and a row stride that are multiples of 8")
        out = torch.empty(M, N, dtype=out_dtype, device=x.device)
        for m0 in range(0, M, 65535 * 64):
            m = min(65535 * 64, M - m0)
            check(lib.fmsamd_gemm_bf16_any(x[m0:].data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), bcode,
                                           out[m0:].data_ptr(), _code(out_dtype), out.stride(0), m, N, K, _stream()))
        return out
    if M <= SKINNY_FAST_ROWS or (M <= SKINNY_MAX_ROWS and not (allow_library and out_dtype == torch.bfloat16)):
        out = torch.empty(M, N, dtype=out_dtype, device=x.device)
        ws, ws_bytes = _skinny_workspace(M, N, K, x.device)
        check(lib.fmsamd_gemm_skinny_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), bcode, out.data_ptr(),
                                          _code(out_dtype), out.stride(0), M, N, K, _row_scale(row_norm, M), _ptr(ws),
                                          ws_bytes, _stream()))
        return out
    if allow_library and out_dtype in (torch.bfloat16, torch.float32):
        # vendor library GEMM, float32 accumulation; float32 results (the logits of many rows) come straight from the
        # accumulators, without a rounding to bfloat16 in between
        if out_dtype == torch.bfloat16:
            out = torch.matmul(x, weight.t())
        else:
            out = torch.mm(x, weight.t(), out_dtype=torch.float32)
        if bias is not None:
            bias_add_(out, bias)
        return out
    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
    check(lib.fmsamd_gemm_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), bcode, out.data_ptr(),
                               _code(out_dtype), out.stride(0), M, N, K, _stream()))
    return out


def linear_into_stream(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    resid: torch.Tensor,
    norm_weight: Optional[torch.Tensor],
    eps: float,
    row_norm: Optional[RowNorm] = None,
):
    """The last product of a residual branch with what follows it (bfloat16, at most SKINNY_FAST_ROWS rows):
    resid += x W^T (+ bias) in float32 in place.  Returns (scaled, RowNorm): scaled = resid * norm_weight in
    bfloat16 and the sums of squares of resid's rows by tiles of 16 columns, which a product takes as its
    `row_norm` to read the RMS-normed stream without a norm kernel in between."""
    _need_cuda(x, weight, bias, resid, norm_weight)
    _rows2d("x", x)
    _rows2d("resid", resid)
    M, K = x.shape
    N = weight.shape[0]
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or weight.dim() != 2 or weight.shape[1] != K or not weight.is_contiguous():
        raise ValueError(f"linear_into_stream takes bfloat16 x [M, {K}] and a contiguous bfloat16 weight [N, {K}]")
    if M > SKINNY_FAST_ROWS or K % 8 or x.stride(0) % 8:
        raise ValueError(f"linear_into_stream: at most {SKINNY_FAST_ROWS} rows, K and the row stride multiples of 8")
    if resid.dtype != torch.float32 or tuple(resid.shape) != (M, N):
        raise ValueError(f"the residual stream is float32 [{M}, {N}]")
    if bias is not None and (bias.shape != (N,) or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{N}] tensor")
    if norm_weight is not None and (norm_weight.shape != (N,) or not norm_weight.is_contiguous()
                                    or norm_weight.dtype not in (torch.float32, torch.bfloat16)):
        raise ValueError(f"the norm weight is a contiguous float32 or bfloat16 [{N}] tensor")
    scaled = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    lib = load()
    partials = torch.empty(M, lib.fmsamd_gemm_skinny_residual_partials(M, N, K), dtype=torch.float32, device=x.device)
    ws, ws_bytes = _skinny_workspace(M, N, K, x.device)
    check(lib.fmsamd_gemm_skinny_residual_bf16(
        x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias), _code(bias.dtype) if bias is not None else 0,
        resid.data_ptr(), resid.stride(0), _ptr(norm_weight), _code(norm_weight.dtype) if norm_weight is not None else 0,
        scaled.data_ptr(), scaled.stride(0), partials.data_ptr(), partials.shape[1], M, N, K, _row_scale(row_norm, M),
        _ptr(ws), ws_bytes, _stream()))
    return scaled, RowNorm(partials, eps)


def gated_linear(
    x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], activation: str, allow_library: bool = True,
    row_norm: Optional[RowNorm] = None,
) -> torch.Tensor:
    """act(x Wg^T + bg) * (x Wu^T + bu) for weight = [Wg; Wu] stacked [2*hidden, K] -> [M, hidden]."""
    M = x.shape[0]
    if weight.shape[0] % 2:
        raise ValueError("the stacked gate/up weight needs an even number of rows")
    hidden = weight.shape[0] // 2
    if (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and M <= (SKINNY_FAST_ROWS if allow_library else SKINNY_MAX_ROWS)
            and x.dim() == 2 and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0):
        _need_cuda(x, weight, bias)
        _rows2d("x", x)
        K = x.shape[1]
        if weight.shape[1] != K or not weight.is_contiguous():
            raise ValueError("weight must be contiguous [2*hidden, K] with K the width of x")
        if bias is not None and (bias.shape != (2 * hidden,) or not bias.is_contiguous()):
            raise ValueError(f"bias must be a contiguous [{2 * hidden}] tensor")
        out = torch.empty(M, hidden, dtype=torch.bfloat16, device=x.device)
        ws, ws_bytes = _skinny_workspace(M, 2 * hidden, K, x.device)
        check(load().fmsamd_gemm_skinny_gated_bf16(x.data_ptr(), x.stride(0), weight.data_ptr(), _ptr(bias),
                                                   _code(bias.dtype) if bias is not None else 0, out.data_ptr(), BF16,
                                                   out.stride(0), M, hidden, K, ACTIVATIONS[activation],
                                                   _row_scale(row_norm, M), _ptr(ws), ws_bytes, _stream()))
        return out
    if row_norm is not None:
        raise ValueError(f"a deferred row norm goes with the bfloat16 product of at most {SKINNY_FAST_ROWS} rows")
    gu = linear(x, weight, None, allow_library=allow_library)
    return gated_act(gu, bias, activation)


# --------------------------------------------------------------------------
# norms behind a branch, further activations
# --------------------------------------------------------------------------
def norm_add_norm(
    resid: torch.Tensor,
    branch: torch.Tensor,
    branch_weight: Optional[torch.Tensor],
    branch_eps: float,
    weight: Optional[torch.Tensor],
    eps: float,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
    want_out: bool = True,
) -> Optional[torch.Tensor]:
    """resid += branch / rms(branch) * branch_weight (float32, in place unless `rows` is given); returns
    resid / rms(resid) * weight in `out_dtype` (only `rows` if given; None if want_out is False)."""
    _need_cuda(resid, branch, branch_weight, weight, rows)
    if resid.dtype != torch.float32 or resid.dim() != 2 or not resid.is_contiguous():
        raise ValueError("the residual stream must be a contiguous float32 [T, width] tensor")
    T, width = resid.shape
    if branch.shape != resid.shape or not branch.is_contiguous() or branch.dtype != out_dtype:
        raise ValueError(f"branch must be contiguous {tuple(resid.shape)} of {out_dtype}, got {tuple(branch.shape)} {branch.dtype}")
    wdtype = None
    for name, t in (("branch weight", branch_weight), ("weight", weight)):
        if t is not None:
            if t.shape != (width,) or not t.is_contiguous():
                raise ValueError(f"norm {name} must be a contiguous [{width}] tensor, got {tuple(t.shape)}")
            if wdtype is not None and t.dtype != wdtype:
                raise TypeError("the two norm weights must have one dtype")
            wdtype = t.dtype
    if width > 16384:
        raise ValueError(f"norm_add_norm keeps a row of at most 16384 elements, the width is {width}")
    n_out = T
    if rows is not None:
        _need_i32("rows", rows)
        n_out = rows.numel()
    out = torch.empty(n_out, width, dtype=out_dtype, device=resid.device) if want_out else None
    check(load().fmsamd_norm_add_norm(resid.data_ptr(), branch.data_ptr(), _code(out_dtype), _ptr(branch_weight), float(branch_eps),
                                      _ptr(weight), _code(wdtype) if wdtype is not None else 0, float(eps), _ptr(out), _ptr(rows),
                                      n_out, width, _stream()))
    return out


def norm_add_norm_affine(
    resid: torch.Tensor,
    branch: torch.Tensor,
    branch_weight: Optional[torch.Tensor],
    branch_bias: Optional[torch.Tensor],
    branch_eps: float,
    branch_mean: bool,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float,
    use_mean: bool,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
    want_out: bool = True,
) -> Optional[torch.Tensor]:
    """norm_add_norm for norms that may take the mean off and add a shift: with N(v; w, b) = (v - mean) / sqrt(var + eps)
    * w + b (var the mean of the squared deviations; without the mean flag no mean is taken off), resid += N(branch;
    branch_weight, branch_bias) (float32, in place unless `rows` is given); returns N(resid; weight, bias) in `out_dtype`
    (only `rows` if given; None if want_out is False)."""
    _need_cuda(resid, branch, branch_weight, branch_bias, weight, bias, rows)
    if resid.dtype != torch.float32 or resid.dim() != 2 or not resid.is_contiguous():
        raise ValueError("the residual stream must be a contiguous float32 [T, width] tensor")
    T, width = resid.shape
    if branch.shape != resid.shape or not branch.is_contiguous() or branch.dtype != out_dtype:
        raise ValueError(f"branch must be contiguous {tuple(resid.shape)} of {out_dtype}, got {tuple(branch.shape)} {branch.dtype}")
    wdtype = None
    for name, t in (("branch weight", branch_weight), ("branch bias", branch_bias), ("weight", weight), ("bias", bias)):
        if t is not None:
            if t.shape != (width,) or not t.is_contiguous():
                raise ValueError(f"norm {name} must be a contiguous [{width}] tensor, got {tuple(t.shape)}")
            if wdtype is not None and t.dtype != wdtype:
                raise TypeError("the norms' weights and shifts must have one dtype")
            wdtype = t.dtype
    if width > 16384:
        raise ValueError(f"norm_add_norm_affine keeps a row of at most 16384 elements, the width is {width}")
    n_out = T
    if rows is not None:
        _need_i32("rows", rows)
        n_out = rows.numel()
    out = torch.empty(n_out, width, dtype=out_dtype, device=resid.device) if want_out else None
    check(load().fmsamd_norm_add_norm_affine(resid.data_ptr(), branch.data_ptr(), _code(out_dtype), _ptr(branch_weight), _ptr(branch_bias),
                                             float(branch_eps), int(bool(branch_mean)), _ptr(weight), _ptr(bias),
                                             _code(wdtype) if wdtype is not None else 0, float(eps), int(bool(use_mean)), _ptr(out),
                                             _ptr(rows), n_out, width, _stream()))
    return out


def rms_norm_cols(x: torch.Tensor, col0: int, n: int, weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """RMS norm of the columns col0 .. col0 + n of float32 rows -> [T, n] in out_dtype."""
    _need_cuda(x, weight)
    _rows2d("x", x)
    if x.dtype != torch.float32 or col0 < 0 or n <= 0 or col0 + n > x.shape[1]:
        raise ValueError(f"rms_norm_cols takes float32 rows and a run of columns inside them, got {x.dtype} {tuple(x.shape)} [{col0}, {col0 + n})")
    if weight is not None and (weight.shape != (n,) or not weight.is_contiguous()):
        raise ValueError(f"the norm weight must be a contiguous [{n}] tensor")
    out = torch.empty(x.shape[0], n, dtype=out_dtype, device=x.device)
    check(load().fmsamd_rms_norm_cols(x.data_ptr(), x.stride(0), col0, n, _ptr(weight), _code(weight.dtype) if weight is not None else 0,
                                      float(eps), out.data_ptr(), _code(out_dtype), out.stride(0), x.shape[0], _stream()))
    return out


def poly_norm(z: torch.Tensor, coefficients, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """a N(z) + b N(z^2) + c N(z^3) + e for coefficients (a, b, c, e), powers element by element, N a row divided by its
    root mean square: float32 rows [T, n] -> [T, n] in out_dtype."""
    _need_cuda(z)
    _rows2d("z", z)
    if z.dtype != torch.float32:
        raise ValueError("poly_norm takes float32 rows")
    a, b, c, e = (float(v) for v in coefficients)
    out = torch.empty(z.shape[0], z.shape[1], dtype=out_dtype, device=z.device)
    check(load().fmsamd_poly_norm(z.data_ptr(), z.stride(0), z.shape[1], a, b, c, e, float(eps), out.data_ptr(), _code(out_dtype),
                                  out.stride(0), z.shape[0], _stream()))
    return out


CHAIN_NONE, CHAIN_CAST, CHAIN_NORM = 0, 1, 2


def group_norm_chain(resid: torch.Tensor, branch: Optional[torch.Tensor], branch_weight: Optional[torch.Tensor], branch_groups: int,
                     branch_eps: float, act_dtype: torch.dtype, out_mode: int = CHAIN_NONE, weight: Optional[torch.Tensor] = None,
                     groups: int = 1, eps: float = 0.0, rows: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """resid += gnorm(branch) * branch_weight (float32, in place unless `rows` is given; branch None: nothing is added), gnorm
    dividing each of `branch_groups` equal consecutive parts of a row by its own root mean square (0: the branch is added
    as it is).  Returns nothing
    (CHAIN_NONE), the stream in act_dtype (CHAIN_CAST), or gnorm(resid) * weight with `groups` parts (CHAIN_NORM); only
    `rows` if given."""
    _need_cuda(resid, branch, branch_weight, weight, rows)
    if resid.dtype != torch.float32 or resid.dim() != 2 or not resid.is_contiguous():
        raise ValueError("the residual stream must be a contiguous float32 [T, width] tensor")
    T, width = resid.shape
    if branch is not None and (branch.shape != resid.shape or not branch.is_contiguous() or branch.dtype != act_dtype):
        raise ValueError(f"branch must be contiguous {tuple(resid.shape)} of {act_dtype}, got {tuple(branch.shape)} {branch.dtype}")
    for name, t in (("branch weight", branch_weight), ("weight", weight)):
        if t is not None and (t.shape != (width,) or not t.is_contiguous()):
            raise ValueError(f"norm {name} must be a contiguous [{width}] tensor, got {tuple(t.shape)}")
    if branch is not None and branch_groups != 0 and (branch_groups < 1 or width % branch_groups):
        raise ValueError(f"{branch_groups} groups do not divide {width} channels")
    if out_mode == CHAIN_NORM and (groups < 1 or width % groups):
        raise ValueError(f"{groups} groups do not divide {width} channels")
    n_out = T
    if rows is not None:
        _need_i32("rows", rows)
        n_out = rows.numel()
    out = torch.empty(n_out, width, dtype=act_dtype, device=resid.device) if out_mode != CHAIN_NONE else None
    check(load().fmsamd_group_norm_chain(resid.data_ptr(), _ptr(branch), _code(act_dtype), _ptr(branch_weight),
                                         _code(branch_weight.dtype) if branch_weight is not None else 0, int(branch_groups), float(branch_eps),
                                         _ptr(weight), _code(weight.dtype) if weight is not None else 0, int(groups), float(eps),
                                         _ptr(out), int(out_mode), _ptr(rows), n_out, width, _stream()))
    return out


CONV_MAX_TAPS = 8


def short_conv(x: torch.Tensor, col0: int, channels: int, conv_w: torch.Tensor, bias: Optional[torch.Tensor], conv_state: Optional[torch.Tensor],
               seq_of_token: torch.Tensor, slot_ids: torch.Tensor, out_dtype: torch.dtype, add_input: bool = False,
               single_tokens: bool = False) -> torch.Tensor:
    """A causal convolution over time on the channels col0 .. col0 + channels of float32 rows: out[t, c] = (x[t, c] if
    add_input) + bias[c] + sum_j conv_w[c, j] x[t - taps + 1 + j, c] over the sequence's own tokens -> [T, channels] in
    out_dtype.  The inputs before the step come from conv_state [slots, taps - 1, channels] (float32; zeros before a
    sequence's start), which is then moved on to the step's last inputs.  single_tokens: every sequence of the step
    brings exactly one token (a decode step); the kernel that convolves then moves the state on as well."""
    _need_cuda(x, conv_w, bias, conv_state, seq_of_token, slot_ids)
    _rows2d("x", x)
    _need_i32("seq_of_token", seq_of_token)
    _need_i32("slot_ids", slot_ids)
    T = x.shape[0]
    if x.dtype != torch.float32 or col0 < 0 or channels <= 0 or col0 + channels > x.shape[1] or seq_of_token.numel() < T:
        raise ValueError("short_conv takes float32 rows that hold the channels asked for, and a sequence index per token")
    if conv_w.dim() != 2 or conv_w.shape[0] != channels or not conv_w.is_contiguous() or not 1 <= conv_w.shape[1] <= CONV_MAX_TAPS:
        raise ValueError(f"the convolution's weights are contiguous [{channels}, taps], taps at most {CONV_MAX_TAPS}")
    taps = conv_w.shape[1]
    if bias is not None and (tuple(bias.shape) != (channels,) or not bias.is_contiguous() or bias.dtype != conv_w.dtype):
        raise ValueError(f"the convolution's bias is a contiguous [{channels}] tensor of the weights' type")
    if taps > 1 and (conv_state is None or conv_state.dtype != torch.float32 or conv_state.dim() != 3
                     or tuple(conv_state.shape[1:]) != (taps - 1, channels) or not conv_state.is_contiguous()):
        raise ValueError(f"the convolution's state is contiguous float32 [slots, {taps - 1}, {channels}]")
    out = torch.empty(T, channels, dtype=out_dtype, device=x.device)
    view = x[:, col0 : col0 + channels]
    check(load().fmsamd_short_conv(view.data_ptr(), x.stride(0), channels, conv_w.data_ptr(), _ptr(bias), _code(conv_w.dtype), taps,
                                   _ptr(conv_state), seq_of_token.data_ptr(), slot_ids.data_ptr(), int(bool(add_input)), out.data_ptr(),
                                   _code(out_dtype), out.stride(0), T, int(bool(single_tokens)), _stream()))
    return out


def rglru_gates(u: torch.Tensor, ra_t: torch.Tensor, ra_b: torch.Tensor, ri_t: torch.Tensor, ri_b: torch.Tensor, lam: torch.Tensor,
                c: float, seq_of_token: torch.Tensor):
    """The gates of the real-gated linear recurrent unit, from float32 rows u [T, channels]: with block-diagonal Ra, Ri given
    as [blocks, in, out] (each block transposed), a = exp(-c sigmoid(Ra u + ra_b) softplus(lam)) and
    b = sqrt(1 - a^2) sigmoid(Ri u + ri_b) u, both float32 [T, channels]."""
    _need_cuda(u, ra_t, ra_b, ri_t, ri_b, lam, seq_of_token)
    _rows2d("u", u)
    _need_i32("seq_of_token", seq_of_token)
    T, C = u.shape
    if u.dtype != torch.float32 or seq_of_token.numel() < T:
        raise ValueError("rglru_gates takes float32 rows and a sequence index per token")
    if ra_t.dim() != 3 or ra_t.shape[1] != ra_t.shape[2] or ra_t.shape[0] * ra_t.shape[1] != C or ra_t.shape != ri_t.shape \
            or ra_t.dtype != ri_t.dtype or not (ra_t.is_contiguous() and ri_t.is_contiguous()):
        raise ValueError(f"the gates' matrices are contiguous [blocks, n, n] with blocks * n = {C}, of one type")
    for name, t in (("ra_b", ra_b), ("ri_b", ri_b), ("lam", lam)):
        if t.dtype != torch.float32 or tuple(t.shape) != (C,) or not t.is_contiguous():
            raise ValueError(f"{name} is a contiguous float32 [{C}] tensor")
    a = torch.empty(T, C, dtype=torch.float32, device=u.device)
    b = torch.empty(T, C, dtype=torch.float32, device=u.device)
    check(load().fmsamd_rglru_gates(u.data_ptr(), u.stride(0), ra_t.data_ptr(), ra_b.data_ptr(), ri_t.data_ptr(), ri_b.data_ptr(),
                                    _code(ra_t.dtype), lam.data_ptr(), float(c), seq_of_token.data_ptr(), a.data_ptr(), b.data_ptr(), T, C,
                                    ra_t.shape[0], _stream()))
    return a, b


def rglru_scan(a: torch.Tensor, b: torch.Tensor, y: torch.Tensor, activation: str, state: torch.Tensor, seq_starts: torch.Tensor,
               seq_of_token: torch.Tensor, slot_ids: torch.Tensor, n_seqs: int, out_dtype: torch.dtype, zero_rows: bool = False) -> torch.Tensor:
    """S <- a S + b over the tokens of every sequence of the step, from and into state [slots, channels] (float32);
    out[t] = S * activation(y[t]) in out_dtype.  a, b: contiguous float32 [T, channels]; y: float32 rows [T, channels] of
    any stride.  Sequence s owns the token rows seq_starts[s] .. seq_starts[s + 1] and the state of slot_ids[s].
    zero_rows: rows that belong to no sequence come back as zeros."""
    _need_cuda(a, b, y, state, seq_starts, seq_of_token, slot_ids)
    _rows2d("y", y)
    for name, t in (("seq_starts", seq_starts), ("seq_of_token", seq_of_token), ("slot_ids", slot_ids)):
        _need_i32(name, t)
    T, C = a.shape
    for name, t in (("a", a), ("b", b)):
        if t.dtype != torch.float32 or tuple(t.shape) != (T, C) or not t.is_contiguous():
            raise ValueError(f"{name} is contiguous float32 [{T}, {C}]")
    if y.dtype != torch.float32 or tuple(y.shape) != (T, C):
        raise ValueError(f"y is float32 [{T}, {C}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != C or not state.is_contiguous():
        raise ValueError(f"the state is contiguous float32 [slots, {C}]")
    if seq_starts.numel() < n_seqs + 1 or slot_ids.numel() < n_seqs or seq_of_token.numel() < T:
        raise ValueError("the step's index arrays are shorter than its sequences or tokens")
    lib = load()
    chunk = lib.fmsamd_rglru_scan_chunk(T, int(n_seqs))
    if chunk:  # long sequences: chunks of token rows side by side (they cover every row, padding rows come back as zeros)
        out = torch.empty(T, C, dtype=out_dtype, device=a.device)
        ws = torch.empty((2 * -(-T // chunk) + int(n_seqs)) * C, dtype=torch.float32, device=a.device)
        check(lib.fmsamd_rglru_scan_chunked(a.data_ptr(), b.data_ptr(), y.data_ptr(), y.stride(0), ACTIVATIONS[activation], state.data_ptr(),
                                            seq_starts.data_ptr(), seq_of_token.data_ptr(), slot_ids.data_ptr(), out.data_ptr(),
                                            _code(out_dtype), out.stride(0), T, int(n_seqs), C, chunk, ws.data_ptr(), _stream()))
        return out
    out = (torch.zeros if zero_rows else torch.empty)(T, C, dtype=out_dtype, device=a.device)
    check(lib.fmsamd_rglru_scan(a.data_ptr(), b.data_ptr(), y.data_ptr(), y.stride(0), ACTIVATIONS[activation], state.data_ptr(),
                                   seq_starts.data_ptr(), seq_of_token.data_ptr(), slot_ids.data_ptr(), out.data_ptr(), _code(out_dtype),
                                   out.stride(0), int(n_seqs), C, _stream()))
    return out


def activation(x: torch.Tensor, kind: str) -> torch.Tensor:
    """act(x), elementwise, for the activations of ACTIVATIONS."""
    _need_cuda(x)
    if not x.is_contiguous():
        raise ValueError("activation takes a contiguous tensor")
    out = torch.empty_like(x)
    check(load().fmsamd_activate(x.data_ptr(), out.data_ptr(), _code(x.dtype), x.numel(), ACTIVATIONS[kind], _stream()))
    return out


def clamped_gated_act(gu: torch.Tensor, limit: float, alpha: float, shift: float) -> torch.Tensor:
    """[T, 2*hidden] (gate first) -> g' * sigmoid(alpha * g') * (u' + shift) with g' = min(g, limit) and
    u' = clamp(u, -limit, limit)."""
    _need_cuda(gu)
    if gu.dim() != 2 or not gu.is_contiguous() or gu.shape[1] % 2:
        raise ValueError("clamped_gated_act takes a contiguous [T, 2*hidden] tensor")
    T, hidden = gu.shape[0], gu.shape[1] // 2
    out = torch.empty(T, hidden, dtype=gu.dtype, device=gu.device)
    for t0 in range(0, T, 65535):
        n = min(65535, T - t0)
        check(load().fmsamd_clamped_gated_act(gu[t0:].data_ptr(), out[t0:].data_ptr(), _code(gu.dtype), n, hidden, float(limit),
                                              float(alpha), float(shift), _stream()))
    return out


# --------------------------------------------------------------------------
# attention over a latent cache
# --------------------------------------------------------------------------
def _check_latent_cache(cache: torch.Tensor, width: int, dtype: torch.dtype) -> None:
    if cache.dim() != 4 or tuple(cache.shape[1:]) != (1, PAGE_TOKENS, width) or not cache.is_contiguous() or cache.dtype != dtype:
        raise ValueError(f"the latent cache must be contiguous {dtype} [pages, 1, {PAGE_TOKENS}, {width}], got {cache.dtype} {tuple(cache.shape)}")


def _check_latent_values(vt_cache: Optional[torch.Tensor], cache: torch.Tensor, rank: int) -> None:
    if vt_cache is not None and (vt_cache.dim() != 4 or tuple(vt_cache.shape) != (cache.shape[0], 1, rank, PAGE_TOKENS)
                                 or not vt_cache.is_contiguous() or vt_cache.dtype != cache.dtype):
        raise ValueError(f"the transposed latent cache must be contiguous {cache.dtype} [{cache.shape[0]}, 1, {rank}, {PAGE_TOKENS}]")


def latent_attention_fits_mfma(rank: int, rot: int) -> bool:
    """True if the matrix-core kernel of the latent attention takes these sizes (the library says)."""
    return bool(load().fmsamd_latent_attn_mfma_fits(int(rank), int(rot)))


def latent_attention_splits(n_tokens: int, nheads: int, max_context: int) -> int:
    """How many blocks share one (token, 16 heads) of the decode step of the MFMA kernel: enough for some 256 blocks in
    all (one a compute unit), no wave with fewer than two tiles of 32 keys at the context bound, at most 32 (every
    part's result goes through the workspace and is merged)."""
    tiles = n_tokens * -(-nheads // 16)
    return max(1, min(-(-256 // tiles), -(-max_context // 32) // 8, 32))


def _check_tables(cos, sin, rot: int) -> int:
    if rot == 0:
        return 0
    if cos is None or sin is None or cos.dtype != torch.float32 or cos.shape != sin.shape or cos.dim() != 2 or cos.shape[1] * 2 != rot:
        raise ValueError("cos/sin tables must be float32 [max_pos, rot/2]")
    if not (cos.is_contiguous() and sin.is_contiguous()):
        raise ValueError("cos/sin tables must be contiguous")
    return cos.shape[0]


def latent_kv_write(down: torch.Tensor, col0: int, rank: int, rot: int, norm_weight: Optional[torch.Tensor], eps: float,
                    positions, seq_of_token, block_table, cos, sin, cache: torch.Tensor, vt_cache: Optional[torch.Tensor] = None) -> None:
    """From float32 rows whose columns col0 .. col0 + rank + rot hold a token's latent and shared key part: the
    RMS-normed latent and the rotated key part go into the token's row of the latent cache; with vt_cache
    [pages, 1, rank, 64] the latent also goes there, transposed."""
    _need_cuda(down, norm_weight, positions, seq_of_token, block_table, cos, sin, cache, vt_cache)
    _rows2d("down", down)
    T = down.shape[0]
    if down.dtype != torch.float32 or col0 < 0 or col0 + rank + rot > down.shape[1]:
        raise ValueError("latent_kv_write takes float32 rows that hold the latent and the shared key part")
    if norm_weight is not None and (norm_weight.shape != (rank,) or not norm_weight.is_contiguous()):
        raise ValueError(f"the latent's norm weight must be a contiguous [{rank}] tensor")
    _check_batch_index(positions, seq_of_token, block_table, T)
    _check_latent_cache(cache, rank + rot, cache.dtype)
    _check_latent_values(vt_cache, cache, rank)
    max_pos = _check_tables(cos, sin, rot)
    check(load().fmsamd_latent_kv_write(down.data_ptr(), down.stride(0), col0, rank, rot, _ptr(norm_weight),
                                        _code(norm_weight.dtype) if norm_weight is not None else 0, float(eps), positions.data_ptr(),
                                        seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0), _ptr(cos), _ptr(sin),
                                        max_pos, cache.data_ptr(), _ptr(vt_cache), _code(cache.dtype), T, _stream()))


def latent_q_rotate(q: torch.Tensor, qa: torch.Tensor, nheads: int, dim: int, rot: int, rank: int, positions, cos, sin) -> None:
    """The rotated part of every head's query, q[t, h, dim:], rotated into qa[t, h, rank:]."""
    _need_cuda(q, qa, positions, cos, sin)
    _rows2d("q", q)
    _rows2d("qa", qa)
    if q.dtype != qa.dtype or q.shape[0] != qa.shape[0] or q.shape[1] != nheads * (dim + rot) or qa.shape[1] != nheads * (rank + rot):
        raise ValueError("latent_q_rotate: q is [T, H*(dim+rot)] and qa [T, H*(rank+rot)] of one type")
    _need_i32("positions", positions)
    if positions.numel() < q.shape[0]:
        raise ValueError("a position per token is needed")
    max_pos = _check_tables(cos, sin, rot)
    check(load().fmsamd_latent_q_rotate(q.data_ptr(), q.stride(0), _code(q.dtype), nheads, dim, rot, qa.data_ptr(), qa.stride(0), rank,
                                        positions.data_ptr(), _ptr(cos), _ptr(sin), max_pos, q.shape[0], _stream()))


def headwise_linear(x: torch.Tensor, x_head_stride: int, weight: torch.Tensor, y: torch.Tensor, y_head_stride: int,
                    gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[t, h*ys : h*ys + N] = weight[h] @ x[t, h*xs : h*xs + K] for weight [H, N, K]; with `gate` (float32 logits
    [T, >= H], row-major) the result is multiplied by sigmoid(gate[t, h]).  x and y are 2-D rows."""
    _need_cuda(x, weight, y, gate)
    _rows2d("x", x)
    _rows2d("y", y)
    if weight.dim() != 3 or not weight.is_contiguous() or weight.dtype != x.dtype or y.dtype != x.dtype:
        raise ValueError("headwise_linear takes a contiguous weight [H, N, K] of the type of x and y")
    H, N, K = weight.shape
    T = x.shape[0]
    if y.shape[0] != T or x.shape[1] < (H - 1) * x_head_stride + K or y.shape[1] < (H - 1) * y_head_stride + N:
        raise ValueError("headwise_linear: the rows of x or y are too short for the heads")
    if gate is not None and (gate.dtype != torch.float32 or gate.dim() != 2 or gate.stride(1) != 1 or gate.shape[0] != T or gate.shape[1] < H):
        raise ValueError("the gate is float32 [T, >= H] with contiguous rows")
    for t0 in range(0, T, 65535 * 16):
        n = min(65535 * 16, T - t0)
        check(load().fmsamd_headwise_linear(x[t0:].data_ptr(), x.stride(0), x_head_stride, weight.data_ptr(), y[t0:].data_ptr(), y.stride(0),
                                            y_head_stride, _ptr(gate[t0:]) if gate is not None else None, gate.stride(0) if gate is not None else 0,
                                            _code(x.dtype), n, H, N, K, _stream()))
    return y


def latent_attention(qa: torch.Tensor, positions, seq_of_token, block_table, cache: torch.Tensor, sink: Optional[torch.Tensor],
                     nheads: int, rank: int, rot: int, scale: float, window: int = 0, *, decode: bool = False,
                     max_context: int = 0, force_generic: bool = False, vt_cache: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of every token over the latent cache of its sequence: qa [T, H*(rank+rot)] holds every head's
    query in the space of the cache rows; returns sum_j p_j latent_j per head, [T, H*rank].  sink: float32 [H] or None.

    bfloat16 with the transposed latent at hand (vt_cache) and sizes that fit runs the MFMA kernel: for prompts a
    wave per (token, 16 heads); for a decode step (one token a sequence; max_context bounds the contexts) the keys of
    every (token, 16 heads) are dealt over several blocks and merged.  Everything else runs the float32 kernel."""
    _need_cuda(qa, positions, seq_of_token, block_table, cache, sink, vt_cache)
    _rows2d("qa", qa)
    T = qa.shape[0]
    if qa.shape[1] != nheads * (rank + rot):
        raise ValueError(f"qa has {qa.shape[1]} columns, expected {nheads * (rank + rot)}")
    _check_batch_index(positions, seq_of_token, block_table, T)
    _check_latent_cache(cache, rank + rot, qa.dtype)
    if sink is not None and (sink.dtype != torch.float32 or tuple(sink.shape) != (nheads,) or not sink.is_contiguous()):
        raise ValueError(f"the sink is a contiguous float32 [{nheads}] tensor")
    out = torch.empty(T, nheads * rank, dtype=qa.dtype, device=qa.device)
    lib = load()
    _check_latent_values(vt_cache, cache, rank)
    if (qa.dtype == torch.bfloat16 and vt_cache is not None and not force_generic and lib.fmsamd_latent_attn_mfma_fits(rank, rot)
            and qa.stride(0) % 8 == 0):
        if decode and max_context <= 0:
            raise ValueError("decode attention needs max_context (an upper bound of every context length)")
        n_splits = latent_attention_splits(T, nheads, max_context) if decode else 0
        ws_bytes = lib.fmsamd_latent_attn_workspace(T, nheads, rank, n_splits)
        ws = torch.empty(max(ws_bytes // 4, 1), dtype=torch.float32, device=qa.device) if ws_bytes else None
        check(lib.fmsamd_latent_attn_mfma(qa.data_ptr(), qa.stride(0), out.data_ptr(), out.stride(0), _ptr(ws), ws_bytes,
                                          positions.data_ptr(), seq_of_token.data_ptr(), block_table.data_ptr(), block_table.stride(0),
                                          cache.data_ptr(), vt_cache.data_ptr(), _ptr(sink), T, nheads, rank, rot, float(scale),
                                          int(window), n_splits, _stream()))
        return out
    for t0 in range(0, T, 65535):
        n = min(65535, T - t0)
        check(lib.fmsamd_latent_attn_generic(qa[t0:].data_ptr(), qa.stride(0), out[t0:].data_ptr(), out.stride(0), _code(qa.dtype),
                                             positions[t0:].data_ptr(), seq_of_token[t0:].data_ptr(), block_table.data_ptr(),
                                             block_table.stride(0), cache.data_ptr(), _ptr(sink), n, nheads, rank, rot, float(scale),
                                             int(window), _stream()))
    return out


# --------------------------------------------------------------------------
# experts
# --------------------------------------------------------------------------
ROUTE_SCORES = {"softmax": 0, "sigmoid": 1, "sigmoid_normed": 2}


def moe_route(logits: torch.Tensor, n_experts: int, top: int, score: str = "softmax"):
    """float32 logits [T, >= n_experts] -> (int32 ids [T, top], float32 weights [T, top]): the `top` largest logits of
    every token among the first n_experts columns, and their weights: the softmax over those alone ("softmax"), each
    one's sigmoid ("sigmoid"), or the sigmoids divided by their sum ("sigmoid_normed")."""
    _need_cuda(logits)
    _rows2d("logits", logits)
    if logits.dtype != torch.float32 or logits.shape[1] < n_experts:
        raise ValueError("router logits are float32 [T, >= experts]")
    T = logits.shape[0]
    ids = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    weights = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    check(load().fmsamd_moe_route(logits.data_ptr(), logits.stride(0), T, n_experts, top, ROUTE_SCORES[score], ids.data_ptr(),
                                  weights.data_ptr(), _stream()))
    return ids, weights


def moe_route_grouped(logits: torch.Tensor, n_outputs: int, top: int, correction: Optional[torch.Tensor] = None, groups: int = 1,
                      keep: int = 1, scale: float = 1.0):
    """float32 logits [T, >= n_outputs] -> (int32 ids [T, top], float32 weights [T, top]).  s = softmax over the first
    n_outputs columns; an output is chosen by s + correction (float32 [n_outputs]) but weighted by s; the outputs form
    `groups` equal runs of neighbours, a group's score is its largest choice score, and only outputs of the `keep` best
    groups can be chosen; the weights are the chosen s over their sum (+ 1e-20), times `scale`."""
    _need_cuda(logits, correction)
    _rows2d("logits", logits)
    if logits.dtype != torch.float32 or logits.shape[1] < n_outputs:
        raise ValueError("router logits are float32 [T, >= outputs]")
    if correction is not None and (correction.dtype != torch.float32 or tuple(correction.shape) != (n_outputs,) or not correction.is_contiguous()):
        raise ValueError(f"the correction is a contiguous float32 [{n_outputs}] tensor")
    if groups < 1 or n_outputs % groups or not 1 <= keep <= groups or keep * (n_outputs // groups) < top:
        raise ValueError(f"{groups} groups over {n_outputs} outputs with {keep} kept cannot give {top} choices")
    T = logits.shape[0]
    ids = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    weights = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    check(load().fmsamd_moe_route_grouped(logits.data_ptr(), logits.stride(0), T, n_outputs, top, _ptr(correction), groups, keep,
                                          float(scale), ids.data_ptr(), weights.data_ptr(), _stream()))
    return ids, weights


def moe_experts(x: torch.Tensor, ids: torch.Tensor, gate_w: Optional[torch.Tensor], up_w: torch.Tensor, down_w: torch.Tensor,
                limit: float, alpha: float, shift: float, in_scale: Optional[torch.Tensor] = None,
                activation: str = "identity") -> torch.Tensor:
    """Every (token, choice) pair through its expert: float32 [T * top, width], row t * top + j the output of expert
    ids[t, j] for token t.  gate_w, up_w [E, ff, width], down_w [E, width, ff].  in_scale (float32 [T, top]): a factor
    on the expert's input for every pair, applied to the float32 sums of the gate and up products.
    gate_w None: experts without a gate, down(activation(up(x))).  A choice outside 0 .. E - 1 (an expert without
    tensors) runs nothing, and its row is left unwritten."""
    _need_cuda(x, ids, gate_w, up_w, down_w, in_scale)
    gated = gate_w is not None
    if not gated:
        gate_w = up_w
    if in_scale is not None and (in_scale.dtype != torch.float32 or tuple(in_scale.shape) != tuple(ids.shape) or not in_scale.is_contiguous()):
        raise ValueError("in_scale is a contiguous float32 tensor of the shape of ids")
    _rows2d("x", x)
    _need_i32("ids", ids)
    T, top = ids.shape
    E, ff, width = gate_w.shape
    if x.shape != (T, width) or tuple(up_w.shape) != (E, ff, width) or tuple(down_w.shape) != (E, width, ff):
        raise ValueError("moe_experts: x [T, width], gate and up [E, ff, width], down [E, width, ff]")
    for w in (gate_w, up_w, down_w):
        if w.dtype != x.dtype or not w.is_contiguous():
            raise TypeError("the experts' weights are contiguous and of the type of x")
    lib = load()
    n_pairs = T * top
    # tiles of 64 rows where the experts have many rows (prompts) and the matrix-core kernel can load the rows
    wide_ok = x.dtype == torch.bfloat16 and width % 8 == 0 and ff % 8 == 0 and x.stride(0) % 8 == 0
    tile_rows = lib.fmsamd_moe_tile_rows(n_pairs, E, int(wide_ok))
    max_tiles = lib.fmsamd_moe_max_tiles(n_pairs, E, tile_rows)
    order = torch.empty(n_pairs, dtype=torch.int32, device=x.device)
    tiles = torch.empty(max_tiles, 3, dtype=torch.int32, device=x.device)
    check(lib.fmsamd_moe_group(ids.data_ptr(), n_pairs, E, order.data_ptr(), tiles.data_ptr(), max_tiles, tile_rows, _stream()))
    hidden = torch.empty(n_pairs, ff, dtype=x.dtype, device=x.device)
    y = torch.empty(n_pairs, width, dtype=torch.float32, device=x.device)
    code = _code(x.dtype)
    check(lib.fmsamd_moe_experts(0, x.data_ptr(), x.stride(0), gate_w.data_ptr(), up_w.data_ptr() if gated else None, hidden.data_ptr(), code,
                                 order.data_ptr(), tiles.data_ptr(), max_tiles, tile_rows, top, ff, width, float(limit), float(alpha), float(shift),
                                 _ptr(in_scale), ACTIVATIONS[activation], _stream()))
    check(lib.fmsamd_moe_experts(1, hidden.data_ptr(), hidden.stride(0), down_w.data_ptr(), None, y.data_ptr(), code,
                                 order.data_ptr(), tiles.data_ptr(), max_tiles, tile_rows, top, width, ff, float(limit), float(alpha), float(shift),
                                 None, 0, _stream()))
    return y


def moe_combine(y: torch.Tensor, weights: Optional[torch.Tensor], shared: Optional[torch.Tensor], shared_gate: Optional[torch.Tensor],
                out_dtype: torch.dtype, top: int = 0, ids: Optional[torch.Tensor] = None, n_experts: int = 0,
                x_in: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[t] = sum_j weights[t, j] * y[t * top + j] (+ sigmoid(shared_gate[t]) * shared[t]) in out_dtype.
    weights None (then `top` says how many rows a token has): the plain sum.
    shared_gate: a float32 column view [T] (any row stride) of logits, or None for an ungated shared output.
    ids [T, top] with n_experts and x_in [T, width] (of out_dtype): a choice of n_experts or more is an identity
    expert, whose output is the token's row of x_in."""
    _need_cuda(y, weights, shared, shared_gate, ids, x_in)
    if weights is not None:
        T, top = weights.shape
    elif top <= 0 or y.dim() != 2 or y.shape[0] % top:
        raise ValueError("moe_combine without weights needs the number of rows a token has")
    else:
        T = y.shape[0] // top
    if y.dtype != torch.float32 or y.dim() != 2 or y.shape[0] != T * top or not y.is_contiguous() or (
            weights is not None and (not weights.is_contiguous() or weights.dtype != torch.float32)):
        raise ValueError("moe_combine: y is contiguous float32 [T * top, width], weights float32 [T, top]")
    width = y.shape[1]
    if shared is not None and (tuple(shared.shape) != (T, width) or shared.dtype != out_dtype or not shared.is_contiguous()):
        raise ValueError("the shared expert's output is contiguous [T, width] of the output type")
    ldg = 0
    if shared_gate is not None:
        if shared is None or shared_gate.dtype != torch.float32 or shared_gate.dim() != 1 or shared_gate.shape[0] != T:
            raise ValueError("the shared gate is a float32 [T] view and needs a shared output")
        ldg = shared_gate.stride(0)
    if ids is not None:
        _need_i32("ids", ids)
        if tuple(ids.shape) != (T, top) or x_in is None or x_in.dtype != out_dtype or x_in.dim() != 2 or x_in.stride(1) != 1 \
                or tuple(x_in.shape) != (T, width):
            raise ValueError("identity experts need ids [T, top] and the tokens' inputs [T, width] of the output type")
    out = torch.empty(T, width, dtype=out_dtype, device=y.device)
    check(load().fmsamd_moe_combine(y.data_ptr(), _ptr(weights), top, _ptr(shared), _ptr(shared_gate), ldg, out.data_ptr(),
                                    _code(out_dtype), T, width, _ptr(ids), int(n_experts), _ptr(x_in) if ids is not None else None,
                                    x_in.stride(0) if ids is not None else 0, _stream()))
    return out


# --------------------------------------------------------------------------
# steps around attention
# --------------------------------------------------------------------------
def qk_projection_norm(proj: torch.Tensor, nq: int, nk: int, nv: int, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                       eps: float, out_dtype: torch.dtype, seq_of_token: Optional[torch.Tensor] = None, norm_dim: int = 0,
                       v_first: Optional[torch.Tensor] = None, v_lambda: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 rows [q (nq) | k (nk) | v (nv) | ...] -> [T, nq + nk + nv] in out_dtype: q and k each RMS-normed over
    their whole run of columns (all heads at once) times a weight, v as it is.  norm_dim > 0: the norms run over every
    run of norm_dim columns (a head) by itself, with weights of norm_dim entries that all heads share.  v_first (rows
    [T, nv] of out_dtype, any row stride) with v_lambda (one float32 number on the device): the values leave as
    (1 - lambda) v + lambda v_first."""
    _need_cuda(proj, q_weight, k_weight, seq_of_token, v_first, v_lambda)
    norm_dim = int(norm_dim)
    if norm_dim < 0 or (norm_dim and (nq % norm_dim or nk % norm_dim)):
        raise ValueError(f"heads of {norm_dim} do not divide queries ({nq}) and keys ({nk})")
    if v_first is not None:
        _rows2d("v_first", v_first)
        if v_first.dtype != out_dtype or tuple(v_first.shape) != (proj.shape[0], nv):
            raise ValueError(f"v_first is [{proj.shape[0]}, {nv}] of {out_dtype}")
        if v_lambda is None or v_lambda.dtype != torch.float32 or v_lambda.numel() != 1:
            raise ValueError("blended values need their factor as one float32 number on the device")
    _rows2d("proj", proj)
    if proj.dtype != torch.float32 or proj.shape[1] < nq + nk + nv:
        raise ValueError("qk_projection_norm takes float32 rows that hold queries, keys and values")
    wdtype = None
    for n, w in ((norm_dim or nq, q_weight), (norm_dim or nk, k_weight)):
        if w is not None:
            if tuple(w.shape) != (n,) or not w.is_contiguous() or (wdtype is not None and w.dtype != wdtype):
                raise ValueError("the norm weights are contiguous vectors of the projections' sizes and of one type")
            wdtype = w.dtype
    if seq_of_token is not None:
        _need_i32("seq_of_token", seq_of_token)
    out = torch.empty(proj.shape[0], nq + nk + nv, dtype=out_dtype, device=proj.device)
    check(load().fmsamd_qk_projection_norm(proj.data_ptr(), proj.stride(0), nq, nk, nv, _ptr(q_weight), _ptr(k_weight),
                                           _code(wdtype) if wdtype is not None else 0, float(eps), out.data_ptr(), _code(out_dtype),
                                           out.stride(0), _ptr(seq_of_token), proj.shape[0], norm_dim, _ptr(v_first),
                                           v_first.stride(0) if v_first is not None else 0, _ptr(v_lambda), _stream()))
    return out


def gate_mul(x: torch.Tensor, gate: Optional[torch.Tensor], activation: str = "sigmoid", scale: float = 1.0,
             out: Optional[torch.Tensor] = None, group: int = 1) -> torch.Tensor:
    """x * act(gate) * scale, elementwise over rows [T, cols]; gate: float32 logits (a view with contiguous rows) or None;
    out: rows of any stride to write into (default: a new tensor).  group > 1: the gate has one column for every run of
    `group` columns of x (a gate per head)."""
    _need_cuda(x, gate, out)
    _rows2d("x", x)
    T, cols = x.shape
    group = int(group)
    if group < 1 or cols % group:
        raise ValueError(f"runs of {group} columns do not divide {cols}")
    if gate is not None:
        _rows2d("gate", gate)
        if gate.dtype != torch.float32 or tuple(gate.shape) != (T, cols // group):
            raise ValueError(f"the gate is float32 [{T}, {cols // group}]")
    if out is None:
        out = torch.empty(T, cols, dtype=x.dtype, device=x.device)
    _rows2d("out", out)
    if out.dtype != x.dtype or tuple(out.shape) != (T, cols):
        raise ValueError(f"out is [{T}, {cols}] of the type of x")
    check(load().fmsamd_gate_mul(x.data_ptr(), x.stride(0), _ptr(gate), gate.stride(0) if gate is not None else 0, ACTIVATIONS[activation],
                                 float(scale), out.data_ptr(), out.stride(0), _code(x.dtype), T, cols, group, _stream()))
    return out


def cast_cols(x: torch.Tensor, col0: int, n: int, dtype: torch.dtype) -> torch.Tensor:
    """The columns col0 .. col0 + n of float32 rows as a contiguous [T, n] tensor of `dtype` (one kernel, no copy before it)."""
    _need_cuda(x)
    _rows2d("x", x)
    if x.dtype != torch.float32 or col0 < 0 or n <= 0 or col0 + n > x.shape[1]:
        raise ValueError(f"cast_cols takes float32 rows and a run of columns inside them, got {x.dtype} {tuple(x.shape)} [{col0}, {col0 + n})")
    out = torch.empty(x.shape[0], n, dtype=dtype, device=x.device)
    view = x[:, col0 : col0 + n]
    check(load().fmsamd_cast_cols(view.data_ptr(), x.stride(0), out.data_ptr(), _code(dtype), out.stride(0), x.shape[0], n, _stream()))
    return out


def scale_(x: torch.Tensor, s: float) -> torch.Tensor:
    """x *= s in place (contiguous float32)."""
    _need_cuda(x)
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise ValueError("scale_ takes a contiguous float32 tensor")
    check(load().fmsamd_scale_f32(x.data_ptr(), x.numel(), float(s), _stream()))
    return x


# --------------------------------------------------------------------------
# the gated delta rule
# --------------------------------------------------------------------------
DELTA_MAX_TAPS = 8
DELTA_MAX_DIM = 256


def delta_prepare(proj: torch.Tensor, col_b: int, a: torch.Tensor, col_a: int, conv_w: torch.Tensor, a_log: torch.Tensor,
                  dt_bias: torch.Tensor, conv_state: torch.Tensor, seq_of_token: torch.Tensor, slot_ids: torch.Tensor, heads: int,
                  kv_heads: int, dim: int, vdim: int, per_channel: bool, q_scale: float):
    """What the recurrence of a step reads, from the float32 projections of its tokens: (qkv [T, C], beta [T, heads],
    decay [T, heads] or [T, heads*dim], kq [T, kv_heads] = k . q), all float32.  The first C = 2*kv_heads*dim + heads*vdim columns of `proj` pass the
    short causal convolution (conv_w [C, taps]; the inputs before the step come from conv_state [slots, taps-1, C], which
    is then moved on), silu, and q and k become unit vectors per head (q times q_scale); beta = sigmoid(proj[:, col_b:]);
    decay = exp(-exp(a_log) * softplus(a[:, col_a:] + dt_bias))."""
    _need_cuda(proj, a, conv_w, a_log, dt_bias, conv_state, seq_of_token, slot_ids)
    _rows2d("proj", proj)
    _rows2d("a", a)
    _need_i32("seq_of_token", seq_of_token)
    _need_i32("slot_ids", slot_ids)
    T = proj.shape[0]
    C = 2 * kv_heads * dim + heads * vdim
    per = dim if per_channel else 1
    if proj.dtype != torch.float32 or a.dtype != torch.float32 or a.shape[0] != T or seq_of_token.numel() < T:
        raise ValueError("delta_prepare takes float32 rows of projections, one per token")
    if proj.shape[1] < max(C, col_b + heads) or col_b < 0 or col_a < 0 or a.shape[1] < col_a + heads * per:
        raise ValueError("delta_prepare: the rows do not hold the columns asked for")
    if conv_w.dim() != 2 or conv_w.shape[0] != C or not conv_w.is_contiguous() or not 1 <= conv_w.shape[1] <= DELTA_MAX_TAPS:
        raise ValueError(f"the convolution's weights are contiguous [{C}, taps], taps at most {DELTA_MAX_TAPS}")
    taps = conv_w.shape[1]
    if (conv_state.dtype != torch.float32 or conv_state.dim() != 3 or tuple(conv_state.shape[1:]) != (max(taps - 1, 1), C)
            or not conv_state.is_contiguous()):
        raise ValueError(f"the convolution's state is contiguous float32 [slots, {max(taps - 1, 1)}, {C}]")
    for name, t, n in (("a_log", a_log, heads), ("dt_bias", dt_bias, heads * per)):
        if t.dtype != torch.float32 or tuple(t.shape) != (n,) or not t.is_contiguous():
            raise ValueError(f"{name} is a contiguous float32 [{n}] tensor")
    if C * 4 > 64 * 1024:
        raise ValueError(f"{C} convolved channels do not fit one block's shared memory")
    qkv = torch.empty(T, C, dtype=torch.float32, device=proj.device)
    beta = torch.empty(T, heads, dtype=torch.float32, device=proj.device)
    decay = torch.empty(T, heads * per, dtype=torch.float32, device=proj.device)
    kq = torch.empty(T, kv_heads, dtype=torch.float32, device=proj.device)
    check(load().fmsamd_delta_prepare(proj.data_ptr(), proj.stride(0), col_b, a.data_ptr(), a.stride(0), col_a, conv_w.data_ptr(),
                                      _code(conv_w.dtype), taps, a_log.data_ptr(), dt_bias.data_ptr(), conv_state.data_ptr(),
                                      seq_of_token.data_ptr(), slot_ids.data_ptr(), qkv.data_ptr(), beta.data_ptr(), decay.data_ptr(),
                                      kq.data_ptr(), T, heads, kv_heads, dim, vdim, int(bool(per_channel)), float(q_scale), _stream()))
    return qkv, beta, decay, kq


def delta_rule(qkv: torch.Tensor, beta: torch.Tensor, decay: torch.Tensor, kq: torch.Tensor, state: torch.Tensor, seq_starts: torch.Tensor,
               seq_of_token: torch.Tensor, slot_ids: torch.Tensor, n_seqs: int, heads: int, kv_heads: int, dim: int, vdim: int,
               per_channel: bool, single_tokens: bool = False) -> torch.Tensor:
    """The recurrence S = g S; u = beta (v - S^T k); S += k u^T; o = S^T q over the tokens of every sequence of the
    step (kq [T, kv_heads] holds k . q of every token, as delta_prepare leaves it), from and into state [slots, heads, vdim, dim] (float32, S transposed) -> o float32 [T, heads*vdim].
    Sequence b of the step owns the token rows seq_starts[b] .. seq_starts[b + 1] and the state of slot_ids[b].
    single_tokens: every sequence brings one token (a decode step); the kernel then stages for that."""
    _need_cuda(qkv, beta, decay, kq, state, seq_starts, seq_of_token, slot_ids)
    for name, t in (("seq_starts", seq_starts), ("seq_of_token", seq_of_token), ("slot_ids", slot_ids)):
        _need_i32(name, t)
    T = qkv.shape[0]
    C = 2 * kv_heads * dim + heads * vdim
    per = dim if per_channel else 1
    for name, t, cols in (("qkv", qkv, C), ("beta", beta, heads), ("decay", decay, heads * per), ("kq", kq, kv_heads)):
        if t.dtype != torch.float32 or tuple(t.shape) != (T, cols) or not t.is_contiguous():
            raise ValueError(f"{name} is contiguous float32 [{T}, {cols}]")
    if state.dtype != torch.float32 or state.dim() != 4 or tuple(state.shape[1:]) != (heads, vdim, dim) or not state.is_contiguous():
        raise ValueError(f"the state is contiguous float32 [slots, {heads}, {vdim}, {dim}]")
    if dim > DELTA_MAX_DIM:
        raise ValueError(f"the delta rule keeps at most {DELTA_MAX_DIM} key channels a head, not {dim}")
    if seq_starts.numel() < n_seqs + 1 or slot_ids.numel() < n_seqs or seq_of_token.numel() < T:
        raise ValueError("the step's index arrays are shorter than its sequences or tokens")
    out = torch.empty(T, heads * vdim, dtype=torch.float32, device=qkv.device)
    check(load().fmsamd_delta_rule(qkv.data_ptr(), beta.data_ptr(), decay.data_ptr(), kq.data_ptr(), state.data_ptr(), out.data_ptr(),
                                   seq_starts.data_ptr(), seq_of_token.data_ptr(), slot_ids.data_ptr(), n_seqs, heads, kv_heads, dim,
                                   vdim, int(bool(per_channel)), int(bool(single_tokens)), _stream()))
    return out


def gated_head_norm(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, activation: str, heads: int, vdim: int,
                    out_dtype: torch.dtype, seq_of_token: torch.Tensor, scale: float = 1.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """o float32 [T, heads*vdim]: every head divided by its root mean square, times weight [vdim], times act(gate)
    (float32 logits [T, heads*vdim], rows of any stride), times scale -> out_dtype (into `out`, rows of any stride)."""
    _need_cuda(o, gate, weight, seq_of_token, out)
    _rows2d("gate", gate)
    _need_i32("seq_of_token", seq_of_token)
    T = o.shape[0]
    if o.dtype != torch.float32 or tuple(o.shape) != (T, heads * vdim) or not o.is_contiguous():
        raise ValueError(f"o is contiguous float32 [T, {heads * vdim}]")
    if gate.dtype != torch.float32 or tuple(gate.shape) != (T, heads * vdim):
        raise ValueError(f"the gate is float32 [{T}, {heads * vdim}]")
    if tuple(weight.shape) != (vdim,) or not weight.is_contiguous():
        raise ValueError(f"the norm weight is a contiguous [{vdim}] tensor")
    if out is None:
        out = torch.empty(T, heads * vdim, dtype=out_dtype, device=o.device)
    _rows2d("out", out)
    if out.dtype != out_dtype or tuple(out.shape) != (T, heads * vdim):
        raise ValueError(f"out is [{T}, {heads * vdim}] of {out_dtype}")
    check(load().fmsamd_gated_head_norm(o.data_ptr(), gate.data_ptr(), gate.stride(0), weight.data_ptr(), _code(weight.dtype), float(eps),
                                        ACTIVATIONS[activation], float(scale), out.data_ptr(), _code(out_dtype), out.stride(0),
                                        seq_of_token.data_ptr(), T, heads, vdim, _stream()))
    return out


# --------------------------------------------------------------------------
def sample(
    logits: torch.Tensor,
    do_sample: bool,
    temperature: float = 1.0,
    top_k: int = 0,
    rng_state: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """One token per row of float32 logits.  rng_state: int64 [rows, 2] (seed, counter), advanced in place."""
    _need_cuda(logits, rng_state, out)
    _rows2d("logits", logits)
    if logits.dtype != torch.float32:
        raise TypeError("logits are float32")
    rows, vocab = logits.shape
    if do_sample:
        if rng_state is None or rng_state.dtype != torch.int64 or tuple(rng_state.shape) != (rows, 2) or not rng_state.is_contiguous():
            raise ValueError("sampling needs a contiguous int64 [rows, 2] generator state")
        if not (temperature > 0 and math.isfinite(temperature)):
            raise ValueError(f"temperature {temperature} must be positive")
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
    elif out.dtype != torch.int32 or out.numel() < rows or not out.is_contiguous():
        raise ValueError("out must be a contiguous int32 tensor with an entry per row")
    if not do_sample and vocab > 4096:
        lib = load()
        nbytes = lib.fmsamd_argmax_workspace(rows, vocab)
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device=logits.device)
        check(lib.fmsamd_argmax(logits.data_ptr(), logits.stride(0), rows, vocab, ws.data_ptr(), nbytes, out.data_ptr(), _stream()))
        return out
    check(load().fmsamd_sample(logits.data_ptr(), logits.stride(0), rows, vocab, int(bool(do_sample)), float(temperature),
                               int(top_k or 0), _ptr(rng_state), out.data_ptr(), _stream()))
    return out


# --------------------------------------------------------------------------
def measured_peaks(read_mib: int = 1024, repeats: int = 5):
    """(bytes per second of a pure read, bfloat16 matrix flops per second) as measured on this GPU now: the best of
    `repeats` runs of a kernel that only reads a buffer of read_mib MiB, and of one that only issues matrix
    instructions on registers.  Takes about a tenth of a second."""
    lib = load()
    buffer = torch.empty(read_mib << 20, dtype=torch.uint8, device="cuda").zero_()
    out = torch.zeros(4, dtype=torch.float32, device="cuda")
    flops = ctypes.c_double(0.0)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def best_ms(launch):
        launch()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(repeats):
            start.record()
            launch()
            end.record()
            torch.cuda.synchronize()
            best = min(best, start.elapsed_time(end))
        return best

    # the best of a few shapes of each: what the hardware can do, not what one launch shape happens to reach
    read_ms = min(best_ms(lambda b=blocks, c=contiguous: check(lib.fmsamd_probe_read(buffer.data_ptr(), buffer.numel(), b, c, out.data_ptr(), _stream())))
                  for blocks in (1024, 2048, 4096) for contiguous in (0, 1))
    mfma = 0.0
    for large in (0, 1):
        for blocks in (256 * 2, 256 * 4):
            ms = best_ms(lambda: check(lib.fmsamd_probe_mfma(blocks, 512, large, out.data_ptr(), ctypes.byref(flops), _stream())))
            mfma = max(mfma, flops.value / (ms / 1000))
    return buffer.numel() / (read_ms / 1000), mfma
