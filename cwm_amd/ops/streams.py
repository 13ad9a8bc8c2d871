"""Entry points of the kernels for a residual kept as several streams (`csrc/streams.hip`), of the activation
between the products of a feed-forward without a gate (`csrc/rowwise.hip`), and of the norm over a whole query or
key projection fused with rotation and cache write (`csrc/rope_kv.hip`).  Shapes, types and devices are checked on
the host; there is no CPU path."""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Any, Optional, Union

import torch

from . import build as _build

MAX_STREAMS = 8  # csrc/streams.hip: STREAMS_MAX
ACTIVATIONS = {"relu2": 0, "relu": 1, "gelu_tanh": 2, "silu": 3}  # csrc/rowwise.hip: act_value


def _base():
    from . import KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream  # the shared helpers of this package

    return KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream


@dataclass
class RoutedSum:
    """A token's result as a weighted sum of rows that has not been added up: `rows` float32 [rows, D] as the grouped
    product leaves them, `groups` the step's pairs grouped by expert (`ExpertGroups`: the row of every (token,
    choice) pair), `weights` float32 [T, top].  `stream_mix_norm` adds the sum up itself, in the order of a token's
    choices; `combine()` gives it as a tensor, the same bits."""

    rows: torch.Tensor
    groups: Any
    weights: torch.Tensor

    def combine(self) -> torch.Tensor:
        from . import combine_routed

        return combine_routed(self.rows, self.groups, self.weights)


def _coefficients(t: Optional[torch.Tensor], shape: tuple, what: str) -> None:
    KernelError = _base()[0]
    if t is not None and (t.dtype != torch.float32 or tuple(t.shape) != shape or not t.is_contiguous()):
        raise KernelError(f"{what} must be a contiguous float32 tensor of shape {shape}")


def embedding_streams(tokens: torch.Tensor, table: torch.Tensor, streams: int, scale: float = 1.0) -> torch.Tensor:
    """float32 [T, streams * D]: `scale` times the row of `table` ([V, D]) for each of int32 `tokens` [T], once for
    every stream."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(tokens, table)
    _i32(tokens, "tokens")
    if table.dim() != 2 or not table.is_contiguous():
        raise KernelError("embedding table must be a contiguous [V, D] tensor")
    if streams < 1:
        raise KernelError("a residual has at least one stream")
    out = torch.empty((tokens.numel(), streams * table.shape[1]), dtype=torch.float32, device=table.device)
    lib = _build.load("streams")
    _check(
        lib,
        lib.cwm_embedding_streams(
            _ptr(out), _ptr(table), ctypes.c_int(_code(table.dtype)), _ptr(tokens), ctypes.c_int(tokens.numel()),
            ctypes.c_int(table.shape[1]), ctypes.c_int(table.shape[0]), ctypes.c_int(streams), ctypes.c_float(scale), _stream(),
        ),
    )
    return out


def stream_mix_norm(
    x: torch.Tensor,
    streams: int,
    y: Union[torch.Tensor, RoutedSum, None],
    mix: Optional[torch.Tensor],
    out_coef: Optional[torch.Tensor],
    in_coef: Optional[torch.Tensor],
    weight: torch.Tensor,
    eps: float,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """`x` is the residual as `streams` vectors a token, float32 [T, streams * D].  If a sublayer's result `y` ([T, D],
    or float32 partial sums [P, T, D], added in order, or a `RoutedSum`) is pending, every stream first becomes
    x_t <- sum_s mix[s, t] x_s + out_coef[t] y, in place.  Returned, in `out_dtype`: the rows
    u / sqrt(mean(u^2) + eps) * weight with u = sum_t in_coef[t] x_t.  `mix` [S, S], `out_coef` [S], `in_coef` [S]:
    float32, None for the identity and ones.  With `rows` (int32 [R]) only those rows are read and `x` stays as it
    is (what is normalised is still the row after the pending change)."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    routed = None
    if isinstance(y, RoutedSum):
        routed, y = y, y.rows
        _need_gpu(routed.weights, routed.groups.pair_row)
    _need_gpu(x, y, mix, out_coef, in_coef, weight, rows)
    if x.dtype != torch.float32 or x.dim() != 2 or not x.is_contiguous() or streams < 1 or x.shape[1] % streams != 0:
        raise KernelError(f"the residual must be a contiguous float32 [T, {streams} * D] tensor")
    if streams > MAX_STREAMS:
        raise KernelError(f"{streams} streams: the kernel takes up to {MAX_STREAMS}")
    n_tokens, dim = x.shape[0], x.shape[1] // streams
    n_partials = 1
    if routed is not None:
        top = routed.groups.top
        if y.dtype != torch.float32 or y.dim() != 2 or y.shape[1] != dim or not y.is_contiguous():
            raise KernelError(f"the experts' rows must be a contiguous float32 [rows, {dim}] tensor")
        if routed.weights.dtype != torch.float32 or tuple(routed.weights.shape) != (n_tokens, top) or not routed.weights.is_contiguous():
            raise KernelError(f"the weights of a weighted sum must be float32 [{n_tokens}, {top}]")
        if routed.groups.pair_row.numel() != n_tokens * top:
            raise KernelError("the list of rows does not fit the tokens")
    elif y is not None:
        if y.dim() == 3:
            if y.dtype != torch.float32:
                raise KernelError("partial sums must be float32")
            n_partials = y.shape[0]
        if tuple(y.shape[-2:]) != (n_tokens, dim) or not y.is_contiguous():
            raise KernelError(f"the sublayer's result {tuple(y.shape)} does not fit {n_tokens} rows of {dim}")
    _coefficients(mix, (streams, streams), "the streams' mixing matrix")
    _coefficients(out_coef, (streams,), "the streams' output coefficients")
    _coefficients(in_coef, (streams,), "the streams' input coefficients")
    _coefficients(weight, (dim,), "the norm's weight")
    if rows is not None:
        _i32(rows, "rows")
    n_out = n_tokens if rows is None else rows.numel()
    out = torch.empty((n_out, dim), dtype=out_dtype, device=x.device)
    lib = _build.load("streams")
    _check(
        lib,
        lib.cwm_stream_mix_norm(
            _ptr(x), ctypes.c_int(streams), _ptr(y), ctypes.c_int(_code(y.dtype) if y is not None else 0), ctypes.c_int(n_partials),
            ctypes.c_long(n_tokens * dim), _ptr(mix), _ptr(out_coef), _ptr(in_coef), _ptr(weight), _ptr(out), ctypes.c_int(_code(out_dtype)),
            _ptr(rows), ctypes.c_int(n_out), ctypes.c_int(dim), ctypes.c_float(eps),
            _ptr(routed.groups.pair_row if routed is not None else None), _ptr(routed.weights if routed is not None else None),
            ctypes.c_int(routed.groups.top if routed is not None else 0), _stream(),
        ),
    )
    return out


def act_rows(x: torch.Tensor, kind: str, out_dtype: torch.dtype) -> torch.Tensor:
    """act(x) element by element in float32, rounded once to `out_dtype`: `x` is [T, F], or float32 partial sums
    [P, T, F] that are added in order first.  `kind`: one of `ACTIVATIONS` ("relu2" is the square of relu)."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(x)
    if kind not in ACTIVATIONS:
        raise KernelError(f"unknown activation {kind!r}; known: {', '.join(ACTIVATIONS)}")
    if x.dim() not in (2, 3) or not x.is_contiguous() or (x.dim() == 3 and x.dtype != torch.float32):
        raise KernelError("act_rows takes a contiguous [T, F] tensor or float32 partial sums [P, T, F]")
    n_partials = x.shape[0] if x.dim() == 3 else 1
    shape = tuple(x.shape[-2:])
    out = torch.empty(shape, dtype=out_dtype, device=x.device)
    lib = _build.load("rowwise")
    _check(
        lib,
        lib.cwm_act_rows(
            _ptr(out), ctypes.c_int(_code(out_dtype)), _ptr(x), ctypes.c_int(_code(x.dtype)), ctypes.c_int(n_partials),
            ctypes.c_long(shape[0] * shape[1]), ctypes.c_int(ACTIVATIONS[kind]), _stream(),
        ),
    )
    return out


def qk_norm_rope_write(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    qk_dim: int,
    v_dim: int,
    head_dim: int,
    q_weight: Optional[torch.Tensor],
    k_weight: Optional[torch.Tensor],
    eps: float,
    positions: torch.Tensor,
    inv_freq: Optional[torch.Tensor],
    out_dtype: torch.dtype,
    cache: Optional[torch.Tensor] = None,
    block_table: Optional[torch.Tensor] = None,
    seq_of_token: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """From the joined projection `qkv` ([T, Hq * qk_dim + Hkv * qk_dim + Hkv * v_dim], or float32 partial sums
    [P, T, ...] of it): queries and keys are each divided by the root mean square of their whole projection (eps
    inside the root) and multiplied by `q_weight` / `k_weight` (float32, one value an element; None: no norm), their
    heads rotated by positions * inv_freq (float32 [head_dim / 2], adjacent pairs, a frequency of 0 leaves its
    pair alone).  Returns the queries [T, Hq, head_dim] in `out_dtype` (elements from qk_dim on are zeros); keys and
    values go into the paged `cache` ([pages, 2, Hkv, page * head_dim], zeros beyond qk_dim and v_dim) where one is
    given.  float32 arithmetic."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(qkv, q_weight, k_weight, positions, inv_freq, cache, block_table, seq_of_token)
    width = (n_q_heads + n_kv_heads) * qk_dim + n_kv_heads * v_dim
    n_partials, partial_stride = 1, 0
    if qkv.dim() == 3:
        if qkv.dtype != torch.float32 or not qkv.is_contiguous():
            raise KernelError("partial sums must be a contiguous float32 [P, T, N] tensor")
        n_partials, n_tokens, partial_stride, stride = qkv.shape[0], qkv.shape[1], qkv.shape[1] * qkv.shape[2], qkv.shape[2]
    elif qkv.dim() == 2 and qkv.stride(1) == 1:
        n_tokens, stride = qkv.shape[0], (qkv.stride(0) if qkv.shape[0] > 1 else qkv.shape[1])
    else:
        raise KernelError("the projection must be [T, N] with contiguous rows or partial sums [P, T, N]")
    if qkv.shape[-1] != width:
        raise KernelError(f"the projection has {qkv.shape[-1]} columns, the heads need {width}")
    if head_dim % 2 != 0 or not (1 <= qk_dim <= head_dim and 1 <= v_dim <= head_dim):
        raise KernelError(f"heads of {qk_dim} and {v_dim} do not fit an even cached head of {head_dim}")
    _coefficients(q_weight, (n_q_heads * qk_dim,), "the queries' norm weight")
    _coefficients(k_weight, (n_kv_heads * qk_dim,), "the keys' norm weight")
    _coefficients(inv_freq, (head_dim // 2,), "the rotary table")
    _i32(positions, "positions")
    if positions.numel() != n_tokens:
        raise KernelError("one position per token is needed")
    page_size = num_pages = table_width = 0
    if cache is not None:
        if block_table is None or seq_of_token is None:
            raise KernelError("a cache write needs a block table and the sequence of each token")
        if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[2] != n_kv_heads or cache.shape[3] % head_dim != 0 or not cache.is_contiguous():
            raise KernelError(f"cache {tuple(cache.shape)} does not fit {n_kv_heads} heads of size {head_dim}")
        if cache.dtype != out_dtype:
            raise KernelError("the cache and the queries must have one type")
        _i32(block_table, "block_table")
        _i32(seq_of_token, "seq_of_token")
        if block_table.dim() != 2 or seq_of_token.numel() != n_tokens:
            raise KernelError("block_table must be [B, W] and seq_of_token [T]")
        num_pages, page_size, table_width = cache.shape[0], cache.shape[3] // head_dim, block_table.shape[1]
    q = torch.empty((n_tokens, n_q_heads, head_dim), dtype=out_dtype, device=qkv.device)
    lib = _build.load("rope_kv")
    _check(
        lib,
        lib.cwm_qk_norm_rope_write(
            _ptr(qkv), ctypes.c_int(_code(qkv.dtype)), ctypes.c_long(stride), ctypes.c_int(n_partials), ctypes.c_long(partial_stride),
            _ptr(q), ctypes.c_int(_code(out_dtype)), _ptr(q_weight), _ptr(k_weight), ctypes.c_float(eps),
            _ptr(positions), _ptr(seq_of_token), _ptr(inv_freq), _ptr(cache), _ptr(block_table),
            ctypes.c_int(table_width), ctypes.c_int(page_size), ctypes.c_int(num_pages), ctypes.c_int(n_tokens),
            ctypes.c_int(n_q_heads), ctypes.c_int(n_kv_heads), ctypes.c_int(qk_dim), ctypes.c_int(v_dim), ctypes.c_int(head_dim), _stream(),
        ),
    )
    return q


def head_norm_rope_write(
    qkv: torch.Tensor,
    n_q_heads: int,
    n_kv_heads: int,
    qk_dim: int,
    v_dim: int,
    head_dim: int,
    bias: Optional[torch.Tensor],
    q_weight: Optional[torch.Tensor],
    k_weight: Optional[torch.Tensor],
    eps: float,
    positions: torch.Tensor,
    inv_freq: Optional[torch.Tensor],
    out_dtype: torch.dtype,
    cache: Optional[torch.Tensor] = None,
    block_table: Optional[torch.Tensor] = None,
    seq_of_token: Optional[torch.Tensor] = None,
    v_other: Optional[torch.Tensor] = None,
    v_mix: Optional[torch.Tensor] = None,
    keep_values: bool = False,
):
    """From the joined projection `qkv` ([T, >= Hq * qk_dim + Hkv * qk_dim + Hkv * v_dim] with q, k and v leading each
    row, or float32 partial sums [P, T, ...] of it) plus `bias` (float32, a value a column of q, k and v): every query
    head and every key head is divided by its own root mean square (eps inside the root) and multiplied by `q_weight` /
    `k_weight` (float32 [qk_dim], the same for all heads; None: no norm), then rotated by positions * inv_freq (float32
    [head_dim / 2], adjacent pairs, a frequency of 0 leaves its pair alone).  With `v_other` ([T, Hkv * v_dim] of
    `out_dtype`, rows may lie apart) and `v_mix` (one float32 on the device) the values become (1 - v_mix) v + v_mix
    v_other.  Returns the queries [T, Hq, head_dim] in `out_dtype` (zeros from qk_dim on), and with `keep_values` also
    the values as they were cached, [T, Hkv * v_dim]; keys and values go into the paged `cache`.  float32 arithmetic."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(qkv, bias, q_weight, k_weight, positions, inv_freq, cache, block_table, seq_of_token, v_other, v_mix)
    width = (n_q_heads + n_kv_heads) * qk_dim + n_kv_heads * v_dim
    n_partials, partial_stride = 1, 0
    if qkv.dim() == 3:
        if qkv.dtype != torch.float32 or not qkv.is_contiguous():
            raise KernelError("partial sums must be a contiguous float32 [P, T, N] tensor")
        n_partials, n_tokens, partial_stride, stride = qkv.shape[0], qkv.shape[1], qkv.shape[1] * qkv.shape[2], qkv.shape[2]
    elif qkv.dim() == 2 and qkv.stride(1) == 1:
        n_tokens, stride = qkv.shape[0], (qkv.stride(0) if qkv.shape[0] > 1 else qkv.shape[1])
    else:
        raise KernelError("the projection must be [T, N] with contiguous rows or partial sums [P, T, N]")
    if qkv.shape[-1] < width:
        raise KernelError(f"the projection has {qkv.shape[-1]} columns, the heads need {width}")
    if head_dim % 2 != 0 or not (1 <= qk_dim <= head_dim and 1 <= v_dim <= head_dim):
        raise KernelError(f"heads of {qk_dim} and {v_dim} do not fit an even cached head of {head_dim}")
    _coefficients(bias, (width,), "the projections' bias")
    _coefficients(q_weight, (qk_dim,), "the queries' norm weight")
    _coefficients(k_weight, (qk_dim,), "the keys' norm weight")
    _coefficients(inv_freq, (head_dim // 2,), "the rotary table")
    _i32(positions, "positions")
    if positions.numel() != n_tokens:
        raise KernelError("one position per token is needed")
    page_size = num_pages = table_width = 0
    if cache is not None:
        if block_table is None or seq_of_token is None:
            raise KernelError("a cache write needs a block table and the sequence of each token")
        if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[2] != n_kv_heads or cache.shape[3] % head_dim != 0 or not cache.is_contiguous():
            raise KernelError(f"cache {tuple(cache.shape)} does not fit {n_kv_heads} heads of size {head_dim}")
        if cache.dtype != out_dtype:
            raise KernelError("the cache and the queries must have one type")
        _i32(block_table, "block_table")
        _i32(seq_of_token, "seq_of_token")
        if block_table.dim() != 2 or seq_of_token.numel() != n_tokens:
            raise KernelError("block_table must be [B, W] and seq_of_token [T]")
        num_pages, page_size, table_width = cache.shape[0], cache.shape[3] // head_dim, block_table.shape[1]
    if (v_other is None) != (v_mix is None):
        raise KernelError("another layer's values and their weight come together")
    other_stride = 0
    if v_other is not None:
        if v_other.dim() != 2 or tuple(v_other.shape) != (n_tokens, n_kv_heads * v_dim) or v_other.stride(1) != 1 or v_other.dtype != out_dtype:
            raise KernelError(f"the other layer's values must be [{n_tokens}, {n_kv_heads * v_dim}] of {out_dtype}")
        if v_mix.dtype != torch.float32 or v_mix.numel() != 1:
            raise KernelError("the values' weight is one float32 number on the device")
        other_stride = v_other.stride(0) if n_tokens > 1 else n_kv_heads * v_dim
    q = torch.empty((n_tokens, n_q_heads, head_dim), dtype=out_dtype, device=qkv.device)
    kept = torch.empty((n_tokens, n_kv_heads * v_dim), dtype=out_dtype, device=qkv.device) if keep_values else None
    lib = _build.load("rope_kv")
    _check(
        lib,
        lib.cwm_head_norm_rope_write(
            _ptr(qkv), ctypes.c_int(_code(qkv.dtype)), ctypes.c_long(stride), ctypes.c_int(n_partials), ctypes.c_long(partial_stride),
            _ptr(bias), _ptr(q), ctypes.c_int(_code(out_dtype)), _ptr(q_weight), _ptr(k_weight), ctypes.c_float(eps),
            _ptr(positions), _ptr(seq_of_token), _ptr(inv_freq), _ptr(cache), _ptr(block_table),
            ctypes.c_int(table_width), ctypes.c_int(page_size), ctypes.c_int(num_pages), ctypes.c_int(n_tokens),
            ctypes.c_int(n_q_heads), ctypes.c_int(n_kv_heads), ctypes.c_int(qk_dim), ctypes.c_int(v_dim), ctypes.c_int(head_dim),
            _ptr(v_other), ctypes.c_long(other_stride), _ptr(v_mix), _ptr(kept), _stream(),
        ),
    )
    return (q, kept) if keep_values else q
