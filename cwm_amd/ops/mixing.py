"""Entry points of the kernels of layers whose attention heads exchange their weights, of gated linear attention, of
short input convolutions, of a layer's own token input and of gated activations on rows
(`csrc/attention_talk.hip`, `csrc/linear_attention.hip`, `csrc/short_conv.hip`, `csrc/token_side.hip`, `csrc/rowwise.hip`).
Shapes, types and devices are checked on the host; there is no CPU path."""

from __future__ import annotations

import ctypes
from typing import Any, Optional, Sequence, Tuple

import torch

from . import build as _build

MAX_TALK_HEADS = 64  # csrc/attention_talk.hip: TALK_MAX_HEADS
TALK_SPLIT = 128  # csrc/attention_talk.hip: columns of a block's range of the score table
MAX_SHORT_CONV_TAPS = 16  # csrc/short_conv.hip: SCONV_MAX_TAPS
MAX_GLA_DIM = 256  # csrc/linear_attention.hip: GLA_MAX_DIM
MAX_SIDE_DIM = 256  # csrc/token_side.hip: SIDE_MAX_DIM
MAX_SIDE_ADDENDS = 4  # csrc/token_side.hip: SIDE_MAX_ADDENDS


def _base():
    from . import KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream  # the shared helpers of this package

    return KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream


TALK_LONG_ROWS = 128  # tokens of a portion from which, in bfloat16, scores and weighted values are matrix products
TALK_LONG_CHUNK = 1024  # rows of such a portion that go through the products at a time


def _talking_long(q_rows, out_rows, cache, table_row, pos0, window, scale, sink, talk, lib) -> None:
    """A long portion of one sequence (bfloat16): its keys and values are gathered from the pages, the scores of all
    its heads are one batched product a key/value head, the mixing kernel normalises and mixes them, and a second
    batched product applies the weights to the values."""
    from . import _check, _code, _ptr, _stream

    n, n_q, hd = q_rows.shape
    n_kv, page_size = cache.shape[2], cache.shape[3] // hd
    per = n_q // n_kv
    for r0 in range(0, n, TALK_LONG_CHUNK):
        r1 = min(n, r0 + TALK_LONG_CHUNK)
        m, p_first = r1 - r0, pos0 + r0
        base = 0 if window is None else max(0, p_first - (window - 1))
        n_keys = pos0 + r1 - base
        keys = torch.empty((n_kv, n_keys, hd), dtype=q_rows.dtype, device=q_rows.device)
        values = torch.empty_like(keys)
        _check(
            lib,
            lib.cwm_talking_gather(
                _ptr(cache), ctypes.c_int(_code(cache.dtype)), _ptr(table_row), ctypes.c_int(table_row.numel()), _ptr(keys), _ptr(values),
                ctypes.c_int(n_kv), ctypes.c_int(hd), ctypes.c_int(page_size), ctypes.c_int(cache.shape[0]), ctypes.c_int(base), ctypes.c_int(n_keys), _stream(),
            ),
        )
        grouped = q_rows[r0:r1].reshape(m, n_kv, per, hd).permute(1, 0, 2, 3).reshape(n_kv, m * per, hd)
        scores = torch.bmm(grouped, keys.transpose(1, 2), out_dtype=torch.float32)  # bfloat16 operands, float32 sums as they are
        weights = torch.empty((n_kv, m * per, n_keys), dtype=q_rows.dtype, device=q_rows.device)
        stats = torch.empty((m, n_q, 2), dtype=torch.float32, device=q_rows.device)
        _check(
            lib,
            lib.cwm_talking_mix(
                _ptr(scores), _ptr(weights), ctypes.c_int(_code(weights.dtype)), _ptr(stats), ctypes.c_int(m), ctypes.c_int(n_keys), ctypes.c_int(n_q),
                ctypes.c_int(n_kv), ctypes.c_int(p_first), ctypes.c_int(base), ctypes.c_int(-1 if window is None else window - 1), ctypes.c_float(scale),
                _ptr(sink), _ptr(talk), _stream(),
            ),
        )
        mixed = torch.bmm(weights, values)  # [Hkv, m * per, hd]
        out_rows[r0:r1] = mixed.reshape(n_kv, m, per, hd).permute(1, 0, 2, 3).reshape(m, n_q * hd)


def talking_attention(
    q: torch.Tensor,
    cache: torch.Tensor,
    block_table: torch.Tensor,
    batch: Any,
    window: Optional[int],
    scale: float,
    sink: Optional[torch.Tensor] = None,
    talk: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Causal attention of `q` [T, Hq, hd] over the paged cache ([pages, 2, Hkv, page * hd]) whose heads mix their
    softmax weights: head h applies sum_g talk[h, g] p_g to the values of its own key/value head, with
    p_g = exp(scale q_g . k) / (sum over the `window` keys up to the query's own + exp(sink_g)).  `sink`: float32 [Hq] or
    None; `talk`: float32 [Hq, Hq] or None (no mixing).  `batch`: the step's descriptor (positions, sequence of each
    token, `cu_q`, `kv_len` and the host's `q_lens`, `kv_lens`).  Scores and weights of the step go through a table in
    float32 (`csrc/attention_talk.hip`); portions of `TALK_LONG_ROWS` tokens and more in bfloat16 take the scores and the
    weighted values as matrix products instead.  Returns [T, Hq * hd] in the type of `q`."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(q, cache, block_table, sink, talk)
    if q.dim() != 3 or q.stride(2) != 1 or q.stride(1) != q.shape[2]:
        raise KernelError("q must be [T, Hq, hd] with contiguous heads")
    n_tokens, n_q, hd = q.shape
    if cache.dim() != 4 or cache.shape[1] != 2 or cache.shape[3] % hd != 0 or not cache.is_contiguous() or cache.dtype != q.dtype:
        raise KernelError(f"cache {tuple(cache.shape)} {cache.dtype} does not fit heads of size {hd} of {q.dtype}")
    n_kv = cache.shape[2]
    if n_q > MAX_TALK_HEADS or n_q % n_kv != 0:
        raise KernelError(f"{n_q} query heads on {n_kv} key/value heads: at most {MAX_TALK_HEADS} heads, in equal groups")
    if window is not None and window < 1:
        raise KernelError("a window holds at least the query's own key")
    if sink is not None and (sink.dtype != torch.float32 or sink.shape != (n_q,) or not sink.is_contiguous()):
        raise KernelError(f"the sinks must be a contiguous float32 [{n_q}] tensor")
    if talk is not None and (talk.dtype != torch.float32 or talk.shape != (n_q, n_q) or not talk.is_contiguous()):
        raise KernelError(f"the heads' mixing matrix must be a contiguous float32 [{n_q}, {n_q}] tensor")
    for name in ("positions", "seq_of_token", "cu_q", "kv_len"):
        _i32(getattr(batch, name), name)
    _i32(block_table, "block_table")
    if batch.positions.numel() != n_tokens or batch.seq_of_token.numel() != n_tokens or block_table.dim() != 2:
        raise KernelError("positions and seq_of_token must be [T], block_table [B, W]")
    width = n_q * hd
    lib = _build.load("attention_talk")
    static = getattr(batch, "static", None)
    reach = (lambda keys: keys) if window is None else (lambda keys: min(keys, window - 1))  # keys before a portion's first token that it reads
    token_list, n_rows, out = None, n_tokens, None
    if static is not None:  # a captured step: one token a sequence, as many keys as the capture allows
        columns = reach(static.max_keys - 1) + 1
    else:
        q_lens, kv_lens = batch.q_lens, batch.kv_lens
        long = [b for b, n in enumerate(q_lens) if n >= TALK_LONG_ROWS] if q.dtype == torch.bfloat16 else []
        if long:
            out = torch.empty((n_tokens, width), dtype=q.dtype, device=q.device)
            starts = [0]
            for n in q_lens:
                starts.append(starts[-1] + n)
            for b in long:
                t0, t1 = starts[b], starts[b + 1]
                _talking_long(q[t0:t1], out[t0:t1], cache, block_table[b], kv_lens[b] - q_lens[b], window, scale, sink, talk, lib)
            rest = [t for b, n in enumerate(q_lens) if b not in long for t in range(starts[b], starts[b] + n)]
            if not rest:
                return out
            token_list = torch.tensor(rest, dtype=torch.int32).to(q.device)
            n_rows = len(rest)
        short = [b for b in range(len(q_lens)) if b not in long]
        columns = max(reach(kv_lens[b] - q_lens[b]) + q_lens[b] for b in short)
    columns = -(-max(1, columns) // TALK_SPLIT) * TALK_SPLIT
    scores = torch.empty((n_rows, n_q, columns), dtype=torch.float32, device=q.device)
    weights = torch.empty((n_rows, n_q, columns), dtype=q.dtype, device=q.device)
    stats = torch.empty((n_rows, n_q, 2), dtype=torch.float32, device=q.device)
    partial = torch.empty((columns // TALK_SPLIT, n_rows, width), dtype=torch.float32, device=q.device)
    _check(
        lib,
        lib.cwm_talking_attention(
            _ptr(q), ctypes.c_long(q.stride(0) if n_tokens > 1 else width), ctypes.c_int(_code(q.dtype)), _ptr(cache), _ptr(block_table),
            ctypes.c_int(block_table.shape[1]), _ptr(token_list), _ptr(batch.positions), _ptr(batch.seq_of_token), _ptr(batch.cu_q), _ptr(batch.kv_len),
            ctypes.c_int(n_rows), ctypes.c_int(n_q), ctypes.c_int(n_kv), ctypes.c_int(hd), ctypes.c_int(cache.shape[3] // hd), ctypes.c_int(cache.shape[0]),
            ctypes.c_int(-1 if window is None else window - 1), ctypes.c_float(scale), _ptr(sink), _ptr(talk), ctypes.c_int(columns),
            _ptr(scores), _ptr(weights), _ptr(stats), _ptr(partial), _stream(),
        ),
    )
    from . import sum_partials

    rows = sum_partials(partial, q.dtype)
    if token_list is None:
        return rows
    out.index_copy_(0, token_list.long(), rows)
    return out


GLA_THREADS = 256  # csrc/linear_attention.hip: threads of a walking block
GLA_ROWS = 32  # and the rows of a column of the state that one of them holds at most


def gla_split(dim: int) -> int:
    """Lanes that share a column of a head's state: the fewest (1, 2, 4, 8) that leave a lane at most GLA_ROWS rows."""
    split = 1
    while split < 8 and -(-dim // split) > GLA_ROWS:
        split *= 2
    return split


def gla_rows(dim: int) -> int:
    """Rows of a column of a head's state that one lane holds: a multiple of 4."""
    return -(-(-(-dim // gla_split(dim))) // 4) * 4


def gla_state_elems(heads: int, dim: int, vdim: int) -> int:
    """float32 elements of one request's state of a gated linear attention, in the walking kernel's own order: per
    (head, tile of value columns) the rows a thread holds, [row][thread]."""
    split = gla_split(dim)
    rows, cols = gla_rows(dim), GLA_THREADS // split
    return heads * -(-vdim // cols) * rows * GLA_THREADS


def gla_state_unpack(flat: torch.Tensor, heads: int, dim: int, vdim: int) -> torch.Tensor:
    """S [heads, dim, vdim] of one request's state row (tests read states this way)."""
    split = gla_split(dim)
    rows, cols = gla_rows(dim), GLA_THREADS // split
    n_vt = -(-vdim // cols)
    # [head][tile][row r][column][part]: element (d = part * rows + r, e = tile * cols + column)
    t = flat[: heads * n_vt * rows * GLA_THREADS].reshape(heads, n_vt, rows, cols, split)
    s = t.permute(0, 4, 2, 1, 3).reshape(heads, split * rows, n_vt * cols)
    return s[:, :dim, :vdim]


def gated_linear_attention(
    proj: torch.Tensor, decay_logits: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, batch: Any,
    heads: int, dim: int, vdim: int, tau: float, eps: float, q_scale: Optional[float] = None,
) -> torch.Tensor:
    """Gated linear attention over the step's tokens (`csrc/linear_attention.hip`).  `proj` [T, heads * (2 dim + 2 vdim)]
    holds queries and keys (heads * dim each), then values and the output gate's projection (heads * vdim each);
    `decay_logits` float32 [T, heads * dim] (bias included): a key channel decays by sigmoid(logit)^(1 / tau); `weight`
    float32 [vdim]; `state` float32 [slots, >= gla_state_elems], read and written at the sequences' slots.  Queries are
    multiplied by `q_scale` (default dim ** -0.5).  Returns [T, heads * vdim] in proj's type: every head's result over
    its root mean square, times weight, times silu(gate).  A step's portions are walked token by token, which gives the
    same bits however a sequence is cut; in bfloat16 a step with a portion of more than `sequence.SCAN_SEGMENT` tokens
    runs its portions in segments side by side, the state carried across them, which differs from the walk by float32
    rounding."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(proj, decay_logits, weight, state)
    n_tokens = proj.shape[0]
    width = heads * (2 * dim + 2 * vdim)
    if proj.dim() != 2 or proj.stride(1) != 1 or proj.shape[1] < width or n_tokens != batch.n_tokens:
        raise KernelError(f"the projection {tuple(proj.shape)} must be [{batch.n_tokens}, >= {width}] with contiguous rows")
    if decay_logits.dtype != torch.float32 or tuple(decay_logits.shape) != (n_tokens, heads * dim) or decay_logits.stride(1) != 1:
        raise KernelError(f"the decays' logits must be float32 [{n_tokens}, {heads * dim}]")
    if weight.dtype != torch.float32 or weight.shape != (vdim,) or not weight.is_contiguous():
        raise KernelError(f"the weight must be a contiguous float32 [{vdim}]")
    if dim > MAX_GLA_DIM:
        raise KernelError(f"heads of {dim} rows: the walking kernel takes up to {MAX_GLA_DIM}")
    need = gla_state_elems(heads, dim, vdim)
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < need or not state.is_contiguous():
        raise KernelError(f"the state must be a contiguous float32 [slots, >= {need}] tensor")
    o_raw = torch.empty((n_tokens, heads * vdim), dtype=torch.float32, device=proj.device)
    out = torch.empty((n_tokens, heads * vdim), dtype=proj.dtype, device=proj.device)
    # long portions in bfloat16 run in segments side by side (float32 keeps to the walk, whose bits no cut changes)
    from .sequence import _scan_segments

    segments = _scan_segments(batch, proj.device) if proj.dtype == torch.bfloat16 else None
    seg_local = seg_decay = seg_start = None
    if segments is not None:
        seg_local, seg_decay, seg_start = (torch.empty((segments.shape[0], need), dtype=torch.float32, device=proj.device) for _ in range(3))
    lib = _build.load("linear_attention")
    _check(
        lib,
        lib.cwm_gated_linear_attention(
            _ptr(proj), ctypes.c_long(proj.stride(0) if n_tokens > 1 else proj.shape[1]), ctypes.c_int(_code(proj.dtype)),
            _ptr(decay_logits), ctypes.c_long(decay_logits.stride(0) if n_tokens > 1 else heads * dim), _ptr(weight), _ptr(o_raw), _ptr(out),
            _ptr(state), ctypes.c_long(state.shape[1]), _ptr(batch.state_slots), _ptr(batch.cu_q), ctypes.c_int(state.shape[0]),
            ctypes.c_int(n_tokens), ctypes.c_int(batch.n_seqs), ctypes.c_int(heads), ctypes.c_int(dim), ctypes.c_int(vdim),
            ctypes.c_float(tau), ctypes.c_float(eps), ctypes.c_float(dim ** -0.5 if q_scale is None else q_scale), _ptr(segments),
            ctypes.c_int(segments.shape[0] if segments is not None else 0), _ptr(seg_local), _ptr(seg_decay), _ptr(seg_start), ctypes.c_long(need), _stream(),
        ),
    )
    return out


def short_conv(
    x: torch.Tensor, weights: Sequence[torch.Tensor], state: Optional[torch.Tensor], batch: Any, write_state: bool = True,
) -> Tuple[torch.Tensor, ...]:
    """x + (causal convolution of x over each sequence of the step), a channel at a time, once for each of the one or
    two `weights` (float32 [taps, D], a row a tap, the last row the current token's): `x` [T, D] (rows may lie apart).
    A sequence's last taps - 1 inputs live in its row of `state` (float32 [slots, >= (taps - 1) * D], oldest first):
    read by the portion's first tokens, then replaced (`write_state`).  Returns a [T, D] tensor of x's type a weight."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(x, state, *weights)
    if x.dim() != 2 or x.stride(1) != 1 or x.shape[0] != batch.n_tokens:
        raise KernelError(f"x must be [{batch.n_tokens}, D] with contiguous rows")
    n_tokens, dim = x.shape
    if not 1 <= len(weights) <= 2:
        raise KernelError("one or two convolutions of the same input are taken")
    taps = weights[0].shape[0]
    for w in weights:
        if w.dtype != torch.float32 or tuple(w.shape) != (taps, dim) or not w.is_contiguous():
            raise KernelError(f"a convolution's weight must be a contiguous float32 [{taps}, {dim}] tensor (a row a tap)")
    if not 1 <= taps <= MAX_SHORT_CONV_TAPS:
        raise KernelError(f"{taps} taps are outside 1..{MAX_SHORT_CONV_TAPS}")
    if taps > 1 and (state is None or state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < (taps - 1) * dim or not state.is_contiguous()):
        raise KernelError(f"the state must be a contiguous float32 [slots, >= {(taps - 1) * dim}] tensor")
    outs = tuple(torch.empty((n_tokens, dim), dtype=x.dtype, device=x.device) for _ in weights)
    # a step of single tokens (a decode step) moves the state in the same launch: a token's thread is its channel's only reader
    q_lens = getattr(batch, "q_lens", None)
    mode = 0 if not write_state else (2 if q_lens and max(q_lens) == 1 else 1)
    lib = _build.load("short_conv")
    _check(
        lib,
        lib.cwm_short_conv(
            _ptr(x), ctypes.c_long(x.stride(0) if n_tokens > 1 else dim), ctypes.c_int(_code(x.dtype)), _ptr(weights[0]),
            _ptr(weights[1] if len(weights) > 1 else None), _ptr(outs[0]), _ptr(outs[1] if len(weights) > 1 else None),
            _ptr(state if taps > 1 else None), ctypes.c_long(state.shape[1] if taps > 1 else 0), _ptr(batch.state_slots), _ptr(batch.cu_q),
            _ptr(batch.seq_of_token), ctypes.c_int(state.shape[0] if taps > 1 else 0), ctypes.c_int(n_tokens), ctypes.c_int(batch.n_seqs),
            ctypes.c_int(dim), ctypes.c_int(taps), ctypes.c_int(mode), _stream(),
        ),
    )
    return outs


def token_side(
    h: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor, column0: int, w_gate: torch.Tensor, w_proj_t: torch.Tensor,
    weight: torch.Tensor, eps: float, round_inputs: bool, pending: Any = None,
) -> None:
    """h (float32 [T, D]) += rms(y) * weight with y = w_proj (gelu_tanh(w_gate h) * e), e the columns column0 ..
    column0 + side_dim of the token's row of `table` ([vocab, n]); w_gate [side_dim, D], `w_proj_t` [side_dim, D] (the
    projection [D, side_dim] transposed, which the kernel reads along D) and the table have one type; `weight` float32 [D].  `round_inputs`: h and the gated values are rounded to bfloat16 where
    they enter the two products.  float32 sums, activation and norm."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(h, tokens, table, w_gate, w_proj_t, weight)
    if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
        raise KernelError("the residual stream must be a contiguous float32 [T, D] tensor")
    n_tokens, dim = h.shape
    _i32(tokens, "tokens")
    if tokens.numel() != n_tokens:
        raise KernelError("one token per row is needed")
    if w_gate.dim() != 2 or w_gate.shape[1] != dim or not w_gate.is_contiguous():
        raise KernelError(f"the gate's weight must be a contiguous [side_dim, {dim}] tensor")
    side_dim = w_gate.shape[0]
    if tuple(w_proj_t.shape) != (side_dim, dim) or not w_proj_t.is_contiguous():
        raise KernelError(f"the projection's weight must be handed over transposed, a contiguous [{side_dim}, {dim}] tensor")
    if table.dim() != 2 or table.stride(1) != 1 or column0 < 0 or column0 + side_dim > table.shape[1]:
        raise KernelError(f"the table {tuple(table.shape)} has no columns {column0}..{column0 + side_dim - 1}")
    if not (table.dtype == w_gate.dtype == w_proj_t.dtype):
        raise KernelError("the table and the two weights must have one type")
    if weight.dtype != torch.float32 or weight.shape != (dim,) or not weight.is_contiguous():
        raise KernelError(f"the norm's weight must be a contiguous float32 [{dim}] tensor")
    if side_dim > MAX_SIDE_DIM:
        raise KernelError(f"{side_dim} side values: the kernel takes up to {MAX_SIDE_DIM}")
    from .sequence import ScaledSum

    terms = [] if pending is None else (pending.terms if isinstance(pending, ScaledSum) else [(pending, 1.0)])
    if len(terms) > MAX_SIDE_ADDENDS:
        raise KernelError(f"{len(terms)} addends: the kernel takes up to {MAX_SIDE_ADDENDS}")
    n = max(1, len(terms))
    ptrs, dtypes, lds, partials = (ctypes.c_void_p * n)(), (ctypes.c_int * n)(), (ctypes.c_long * n)(), (ctypes.c_int * n)()
    strides, scales = (ctypes.c_long * n)(), (ctypes.c_float * n)()
    for i, (t, c) in enumerate(terms):
        _need_gpu(t)
        if t.dim() == 3:
            if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape[1:]) != (n_tokens, dim):
                raise KernelError(f"partial sums {tuple(t.shape)} must be contiguous float32 [P, {n_tokens}, {dim}]")
            partials[i], strides[i], lds[i] = t.shape[0], n_tokens * dim, dim
        else:
            if t.dim() != 2 or t.stride(1) != 1 or tuple(t.shape) != (n_tokens, dim):
                raise KernelError(f"an addend {tuple(t.shape)} does not match the residual stream {tuple(h.shape)}")
            partials[i], strides[i], lds[i] = 1, 0, (t.stride(0) if n_tokens > 1 else dim)
        ptrs[i], dtypes[i], scales[i] = t.data_ptr(), _code(t.dtype), c
    lib = _build.load("token_side")
    _check(
        lib,
        lib.cwm_token_side(
            _ptr(h), _ptr(tokens), _ptr(table), ctypes.c_long(table.stride(0)), ctypes.c_int(column0), _ptr(w_gate), _ptr(w_proj_t),
            ctypes.c_int(_code(table.dtype)), _ptr(weight), ctypes.c_int(n_tokens), ctypes.c_int(dim), ctypes.c_int(side_dim),
            ctypes.c_int(table.shape[0]), ctypes.c_float(eps), ctypes.c_int(int(round_inputs)), ctypes.c_int(len(terms)), ptrs, dtypes, lds,
            partials, strides, scales, _stream(),
        ),
    )


def gated_act_rows(x: torch.Tensor, hidden: int, activation: Any, out_dtype: torch.dtype, row_gate_col: Optional[int] = None) -> torch.Tensor:
    """What a gated feed-forward makes of its joined product `x` ([T, >= 2 hidden] with a row's gate values first, then
    its up values; or float32 partial sums [P, T, n], added in order first): `activation` is an `ops.GatedActivation`.
    With `row_gate_col` every row is also multiplied by the sigmoid of that column of x.  float32 arithmetic, rounded
    once; returns [T, hidden] of `out_dtype`."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(x)
    if x.dim() == 3:
        if x.dtype != torch.float32 or not x.is_contiguous():
            raise KernelError("partial sums must be a contiguous float32 [P, T, n] tensor")
        n_partials, n_rows, n = x.shape
        ld, partial_stride = n, n_rows * n
    elif x.dim() == 2 and x.stride(1) == 1:
        n_partials, (n_rows, n) = 1, x.shape
        ld, partial_stride = (x.stride(0) if n_rows > 1 else n), 0
    else:
        raise KernelError("gated_act_rows takes [T, n] with contiguous rows or float32 partial sums [P, T, n]")
    if n < 2 * hidden or (row_gate_col is not None and not 0 <= row_gate_col < n):
        raise KernelError(f"rows of {n} values do not hold a gate and an up part of {hidden} each (and the row's gate)")
    out = torch.empty((n_rows, hidden), dtype=out_dtype, device=x.device)
    lib = _build.load("rowwise")
    _check(
        lib,
        lib.cwm_gated_act_rows(
            _ptr(out), ctypes.c_int(_code(out_dtype)), _ptr(x), ctypes.c_int(_code(x.dtype)), ctypes.c_long(ld), ctypes.c_int(n_partials),
            ctypes.c_long(partial_stride), ctypes.c_int(n_rows), ctypes.c_int(hidden), ctypes.c_int(-1 if row_gate_col is None else row_gate_col),
            ctypes.c_int(activation.code()), ctypes.c_float(activation.alpha), ctypes.c_float(activation.limit), _stream(),
        ),
    )
    return out
