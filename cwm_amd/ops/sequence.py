"""Entry points of the row-wise and sequential kernels of layers with group norms, token shift, a selective
state space and gates (`csrc/groupnorm.hip`, `csrc/state_space.hip`).  Shapes, types and devices are checked on
the host; there is no CPU path."""

from __future__ import annotations

import ctypes
from typing import Any, Optional

import torch

from . import build as _build

MAX_CONV_TAPS = 8  # csrc/state_space.hip: CONV_MAX_TAPS
MAX_SSM_STATE = 256  # csrc/state_space.hip: SCAN_ROWS * 16


def _base():
    from . import KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream  # the shared helpers of this package

    return KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream


def _rows_2d(t: torch.Tensor, what: str) -> None:
    KernelError = _base()[0]
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{what} must be [rows, n] with contiguous rows, found {tuple(t.shape)} with strides {t.stride()}")


def group_rmsnorm(
    x: torch.Tensor,
    weight: torch.Tensor,
    groups: int,
    eps: float,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
    out: Optional[torch.Tensor] = None,
    accumulate: bool = False,
    gate: Optional[torch.Tensor] = None,
    copy: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """weight * x_g / sqrt(mean(x_g^2) + eps) for each of `groups` equal consecutive parts x_g of every row, float32
    arithmetic.  `x` is [T, D] (rows may lie apart) or float32 partial sums [P, T, D], added in order first; with
    `gate` ([T, D]) the row is multiplied by silu(gate) before the norm.  `rows` (int32 [R]) chooses rows.  The
    result goes to a new [R, D] tensor of `out_dtype`, or into `out` ([R, D], which may be `x` itself), added to what
    is there if `accumulate`.  `copy` (contiguous [R, D] of any type) also receives the rows as `out` then holds them."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(x, weight, rows, out, gate, copy)
    n_partials, partial_stride = 1, 0
    if x.dim() == 3:
        if x.dtype != torch.float32 or not x.is_contiguous():
            raise KernelError("partial sums must be a contiguous float32 [P, T, D] tensor")
        n_partials, partial_stride = x.shape[0], x.shape[1] * x.shape[2]
        n_tokens, dim, src_ld = x.shape[1], x.shape[2], x.shape[2]
    else:
        _rows_2d(x, "x")
        n_tokens, dim = x.shape
        src_ld = x.stride(0) if n_tokens > 1 else dim
    if weight.shape != (dim,) or not weight.is_contiguous():
        raise KernelError(f"norm weight has shape {tuple(weight.shape)}, expected ({dim},)")
    if groups < 1 or dim % groups != 0:
        raise KernelError(f"{dim} elements do not divide into {groups} groups")
    if rows is not None:
        _i32(rows, "rows")
    n_out = n_tokens if rows is None else rows.numel()
    if out is None:
        if accumulate:
            raise KernelError("accumulate needs a tensor to add into")
        out = torch.empty((n_out, dim), dtype=out_dtype, device=x.device)
    else:
        _rows_2d(out, "out")
        if tuple(out.shape) != (n_out, dim):
            raise KernelError(f"out {tuple(out.shape)} does not fit {n_out} rows of {dim}")
    gate_ld = 0
    if gate is not None:
        _rows_2d(gate, "gate")
        if tuple(gate.shape) != (n_tokens, dim):
            raise KernelError(f"gate {tuple(gate.shape)} does not fit x")
        gate_ld = gate.stride(0) if n_tokens > 1 else dim
    if copy is not None and (tuple(copy.shape) != (n_out, dim) or not copy.is_contiguous()):
        raise KernelError(f"copy {tuple(copy.shape)} must be a contiguous [{n_out}, {dim}] tensor")
    lib = _build.load("groupnorm")
    _check(
        lib,
        lib.cwm_group_norm(
            _ptr(x), ctypes.c_int(_code(x.dtype)), ctypes.c_long(src_ld), ctypes.c_int(n_partials), ctypes.c_long(partial_stride),
            _ptr(gate), ctypes.c_int(_code(gate.dtype) if gate is not None else 0), ctypes.c_long(gate_ld),
            _ptr(weight), ctypes.c_int(_code(weight.dtype)), _ptr(out), ctypes.c_int(_code(out.dtype)),
            ctypes.c_long(out.stride(0) if n_out > 1 else dim), _ptr(rows), ctypes.c_int(n_out), ctypes.c_int(dim), ctypes.c_int(groups),
            ctypes.c_float(eps), ctypes.c_int(int(accumulate)), _ptr(copy), ctypes.c_int(_code(copy.dtype) if copy is not None else 0),
            ctypes.c_long(dim), _stream(),
        ),
    )
    return out


def add_rows(h: torch.Tensor, delta: torch.Tensor) -> None:
    """h (float32 [T, D]) += delta ([T, D], or partial sums [P, T, D] added in order)."""
    if delta.dim() == 3:
        for p in range(delta.shape[0]):
            h.add_(delta[p])
    else:
        h.add_(delta)


def cast_rows(h: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """The float32 rows in `dtype` (the rows themselves if that is float32)."""
    if h.dtype == dtype:
        return h
    from . import sum_partials

    return sum_partials(h.unsqueeze(0), dtype)


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, batch: Any, out_dtype: torch.dtype, write_state: bool = True) -> torch.Tensor:
    """s_t = h_t + (h_(t-1) - h_t) * mu for the step's tokens: `h` float32 [T, D]; the row before a portion's first
    token is the sequence's row of `state` (float32 [slots, D]; zero at position 0), which then receives the
    portion's last row."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(h, mu, state)
    if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
        raise KernelError("the stream must be a contiguous float32 [T, D] tensor")
    n_tokens, dim = h.shape
    if mu.dtype != torch.float32 or mu.shape != (dim,) or not mu.is_contiguous():
        raise KernelError(f"mu must be float32 [{dim}]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != dim or not state.is_contiguous():
        raise KernelError(f"the state must be float32 [slots, {dim}]")
    if n_tokens != batch.n_tokens:
        raise KernelError("one row per token of the step is needed")
    out = torch.empty((n_tokens, dim), dtype=out_dtype, device=h.device)
    lib = _build.load("groupnorm")
    _check(
        lib,
        lib.cwm_token_shift(
            _ptr(h), _ptr(mu), _ptr(state), _ptr(batch.state_slots), _ptr(batch.cu_q), _ptr(batch.seq_of_token), _ptr(batch.positions),
            _ptr(out), ctypes.c_int(_code(out_dtype)), ctypes.c_int(n_tokens), ctypes.c_int(dim), ctypes.c_int(state.shape[0]),
            ctypes.c_int(int(write_state)), _stream(),
        ),
    )
    return out


def sigmoid_mul(a: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """a * sigmoid(gate), both [T, n] of one type (rows may lie apart); float32 arithmetic."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(a, gate)
    _rows_2d(a, "a")
    _rows_2d(gate, "gate")
    if a.shape != gate.shape or a.dtype != gate.dtype:
        raise KernelError(f"a {tuple(a.shape)} {a.dtype} and gate {tuple(gate.shape)} {gate.dtype} do not match")
    n, width = a.shape
    out = torch.empty((n, width), dtype=a.dtype, device=a.device)
    lib = _build.load("groupnorm")
    _check(
        lib,
        lib.cwm_sigmoid_mul(
            _ptr(a), ctypes.c_long(a.stride(0) if n > 1 else width), _ptr(gate), ctypes.c_long(gate.stride(0) if n > 1 else width),
            _ptr(out), ctypes.c_long(width), ctypes.c_int(_code(a.dtype)), ctypes.c_int(n), ctypes.c_int(width), _stream(),
        ),
    )
    return out


def causal_conv_silu(
    x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, state: torch.Tensor, state_offset: int, batch: Any,
    weight_by_tap: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """silu(bias + causal convolution) per channel over each sequence of the step: `x` [T, C] (rows may lie apart),
    `weight` float32 [C, taps] (the last column is the current token's), `bias` float32 [C].  A sequence's last
    taps - 1 inputs live in its row of `state` (float32 [slots, n]) from `state_offset` on, [taps - 1, C] oldest
    first: read by the portion's first tokens, then replaced.  Returns [T, C] in the type of `x`."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(x, weight, bias, state)
    _rows_2d(x, "x")
    n_tokens, channels = x.shape
    if weight.dtype != torch.float32 or weight.dim() != 2 or weight.shape[0] != channels or not weight.is_contiguous():
        raise KernelError(f"the convolution's weight must be float32 [{channels}, taps]")
    taps = weight.shape[1]
    if bias.dtype != torch.float32 or bias.shape != (channels,) or not bias.is_contiguous():
        raise KernelError(f"the convolution's bias must be float32 [{channels}]")
    if state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous():
        raise KernelError("the state must be a contiguous float32 [slots, n] tensor")
    if state_offset < 0 or state_offset + (taps - 1) * channels > state.shape[1]:
        raise KernelError("the state row does not hold the convolution's inputs")
    if n_tokens != batch.n_tokens:
        raise KernelError("one row per token of the step is needed")
    out = torch.empty((n_tokens, channels), dtype=x.dtype, device=x.device)
    lib = _build.load("state_space")
    _check(
        lib,
        lib.cwm_conv_silu(
            _ptr(x), ctypes.c_long(x.stride(0) if n_tokens > 1 else channels), ctypes.c_int(_code(x.dtype)), _ptr(weight), _ptr(weight_by_tap), _ptr(bias),
            _ptr(state), ctypes.c_long(state.shape[1]), ctypes.c_long(state_offset), _ptr(batch.state_slots), _ptr(batch.cu_q),
            _ptr(batch.seq_of_token), _ptr(out), ctypes.c_int(n_tokens), ctypes.c_int(batch.n_seqs), ctypes.c_int(channels), ctypes.c_int(taps),
            ctypes.c_int(state.shape[0]), _stream(),
        ),
    )
    return out


SCAN_ROWS = 16  # csrc/state_space.hip: rows of a head's state that one thread holds


def scan_split(n_state: int) -> int:
    """Lanes that share a column of a head's state (csrc/state_space.hip: cwm_scan_split)."""
    split = 1
    while split * SCAN_ROWS < n_state:
        split *= 2
    return split


def scan_state_elems(heads: int, head_dim: int, n_state: int) -> int:
    """float32 values that the scan kernel keeps for one request: every head's state padded to 16 * split rows."""
    return heads * SCAN_ROWS * scan_split(n_state) * head_dim


def scan_state_pack(states: torch.Tensor) -> torch.Tensor:
    """[heads, n_state, head_dim] -> the flat order in which the scan kernel keeps it: per head [q][p][s][j] for row
    4 (s + q split) + j of column p, rows from n_state on zero.  (For tests and for looking at a state.)"""
    heads, n_state, head_dim = states.shape
    split = scan_split(n_state)
    padded = torch.zeros((heads, SCAN_ROWS * split, head_dim), dtype=states.dtype, device=states.device)
    padded[:, :n_state] = states
    # row n = 4 (s + q split) + j  ->  [q][s][j]
    return padded.reshape(heads, SCAN_ROWS // 4, split, 4, head_dim).permute(0, 1, 4, 2, 3).reshape(-1).contiguous()


def scan_state_unpack(flat: torch.Tensor, heads: int, head_dim: int, n_state: int) -> torch.Tensor:
    """The inverse of `scan_state_pack`: [heads, n_state, head_dim]."""
    split = scan_split(n_state)
    rows = flat[: scan_state_elems(heads, head_dim, n_state)].reshape(heads, SCAN_ROWS // 4, head_dim, split, 4)
    return rows.permute(0, 1, 3, 4, 2).reshape(heads, SCAN_ROWS * split, head_dim)[:, :n_state].contiguous()


SCAN_SEGMENT = 256  # tokens of a segment; a step with a longer portion runs its portions' segments side by side


def _scan_segments(batch: Any, device: torch.device):
    """The step's list of segments for the scan kernel (int32 [n, 6] on the device: sequence, first token, end token,
    number of the segment in its sequence, the sequence's first scratch entry, segments of the sequence), or None if
    no portion is longer than a segment.  Built once a step from the host's copy of the portions' lengths."""
    q_lens = getattr(batch, "q_lens", None)
    if not q_lens or max(q_lens) <= SCAN_SEGMENT:
        return None
    scratch = getattr(batch, "scratch", None)
    if scratch is not None and "scan_segments" in scratch:
        return scratch["scan_segments"]
    rows, first, base = [], 0, 0
    for b, q in enumerate(q_lens):
        n = -(-q // SCAN_SEGMENT)
        for j in range(n):
            rows.append((b, first + j * SCAN_SEGMENT, first + min(q, (j + 1) * SCAN_SEGMENT), j, base, n))
        first += q
        base += n
    host = torch.tensor(rows, dtype=torch.int32)
    table = (host.pin_memory() if device.type == "cuda" else host).to(device, non_blocking=True)
    if scratch is not None:
        scratch["scan_segments"] = table
    return table


def selective_scan(
    xbc: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, a_log: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, batch: Any,
    heads: int, head_dim: int, n_state: int, groups: int,
) -> torch.Tensor:
    """The recurrence S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x per head over each sequence of the step,
    in float32, from and into the sequences' rows of `state` (float32 [slots, n], n a multiple of 4; S of all heads
    first, `scan_state_elems` values in the kernel's own order, see `scan_state_pack`).  `xbc` [T, heads * head_dim + 2 * groups * n_state] = [x | B | C]; `dt` [T, heads] before
    bias and softplus (rows may lie apart); `dt_bias`, `a_log`, `d_skip` float32 [heads].  Returns y float32
    [T, heads * head_dim].  Portions of up to `SCAN_SEGMENT` tokens are walked token by token, which gives the same
    bits however a sequence is cut; a step with a longer portion (`batch.q_lens`) cuts its portions into segments that
    run side by side and carries the state across them, which differs from the walk by rounding."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(xbc, dt, dt_bias, a_log, d_skip, state)
    _rows_2d(xbc, "xbc")
    _rows_2d(dt, "dt")
    n_tokens = xbc.shape[0]
    inner = heads * head_dim
    if xbc.shape[1] != inner + 2 * groups * n_state or dt.shape != (n_tokens, heads) or dt.dtype != xbc.dtype:
        raise KernelError(f"xbc {tuple(xbc.shape)} and dt {tuple(dt.shape)} do not fit {heads} heads of {head_dim} with {groups} groups of {n_state}")
    for name, t in (("dt_bias", dt_bias), ("A_log", a_log), ("D", d_skip)):
        if t.dtype != torch.float32 or t.shape != (heads,) or not t.is_contiguous():
            raise KernelError(f"{name} must be float32 [{heads}]")
    if (
        state.dtype != torch.float32 or state.dim() != 2 or not state.is_contiguous() or state.shape[1] % 4 != 0
        or state.shape[1] < scan_state_elems(heads, head_dim, n_state)
    ):
        raise KernelError("the state must be a contiguous float32 [slots, n] tensor, n a multiple of 4, that holds every head's state")
    if n_state > MAX_SSM_STATE:
        raise KernelError(f"a state of {n_state} rows is more than the {MAX_SSM_STATE} the scan kernel takes")
    if n_tokens != batch.n_tokens:
        raise KernelError("one row per token of the step is needed")
    y = torch.empty((n_tokens, inner), dtype=torch.float32, device=xbc.device)
    segments = _scan_segments(batch, xbc.device)
    seg_state = seg_decay = None
    if segments is not None:
        if segments.shape[0] > 65535:
            segments = None  # (more segments than one launch counts: the portions are walked whole)
        else:
            seg_state = torch.empty((segments.shape[0], scan_state_elems(heads, head_dim, n_state)), dtype=torch.float32, device=xbc.device)
            seg_decay = torch.empty((segments.shape[0], heads), dtype=torch.float32, device=xbc.device)
    lib = _build.load("state_space")
    _check(
        lib,
        lib.cwm_selective_scan(
            _ptr(xbc), ctypes.c_long(xbc.stride(0) if n_tokens > 1 else xbc.shape[1]), _ptr(dt), ctypes.c_long(dt.stride(0) if n_tokens > 1 else heads),
            ctypes.c_int(_code(xbc.dtype)), _ptr(dt_bias), _ptr(a_log), _ptr(d_skip), _ptr(state), ctypes.c_long(state.shape[1]),
            _ptr(batch.state_slots), _ptr(batch.cu_q), _ptr(y), ctypes.c_int(n_tokens), ctypes.c_int(batch.n_seqs), ctypes.c_int(heads),
            ctypes.c_int(head_dim), ctypes.c_int(n_state), ctypes.c_int(groups), ctypes.c_int(state.shape[0]),
            _ptr(segments), ctypes.c_int(segments.shape[0] if segments is not None else 0), _ptr(seg_state), _ptr(seg_decay), _stream(),
        ),
    )
    return y


# --------------------------------------------------------------------------- #
class ScaledSum:
    """A sum that has not been done yet: `terms` is a list of (tensor, factor), each tensor [T, D] (rows may lie
    apart) or float32 partial sums [P, T, D].  The kernel that reads it next adds the terms up in their order,
    in float32: the results of several sublayers that all join the residual at once."""

    def __init__(self, terms) -> None:
        self.terms = [(t, float(c)) for t, c in terms]

    def total(self, dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """The sum as one tensor (for readers that have no kernel of their own for it)."""
        out = None
        for t, c in self.terms:
            x = (t.sum(dim=0) if t.dim() == 3 else t).to(torch.float32) * c
            out = x if out is None else out + x
        return out.to(dtype)


_ln_limits: Optional[tuple] = None


def layernorm_limits() -> tuple:
    """(most addends, longest row) that `add_layernorm` takes, asked of the kernel library."""
    global _ln_limits
    if _ln_limits is None:
        lib = _build.load("layernorm")
        _ln_limits = (int(lib.cwm_layernorm_max_addends()), int(lib.cwm_layernorm_max_dim()))
    return _ln_limits


def add_layernorm(
    h: torch.Tensor,
    delta: Any,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float,
    out_dtype: torch.dtype,
    rows: Optional[torch.Tensor] = None,
    weight2: Optional[torch.Tensor] = None,
    bias2: Optional[torch.Tensor] = None,
):
    """`h` (float32 [T, D]) += `delta` in place, then the layer norm of its rows, (x - mean) / sqrt(var + eps) * weight
    + bias with the variance taken about the mean, in float32.  `delta`: None, a tensor [T, D], float32 partial sums
    [P, T, D], or a `ScaledSum` of such.  With `weight2` and `bias2` a second norm of the same rows (one mean, one
    variance) is returned beside the first.  With `rows` (int32 [R]) only those rows are normalised and `h` is not
    changed.  Without `weight` only the sum is done and nothing is returned."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(h, weight, bias, rows, weight2, bias2)
    if h.dtype != torch.float32 or h.dim() != 2 or not h.is_contiguous():
        raise KernelError("the residual stream must be a contiguous float32 [T, D] tensor")
    n_tokens, dim = h.shape
    max_addends, max_dim = layernorm_limits()
    if dim > max_dim:
        raise KernelError(f"rows of {dim} elements: the layer norm kernel takes up to {max_dim}")
    terms = [] if delta is None else (delta.terms if isinstance(delta, ScaledSum) else [(delta, 1.0)])
    if len(terms) > max_addends:
        raise KernelError(f"{len(terms)} addends: the layer norm kernel takes up to {max_addends}")
    ptrs = (ctypes.c_void_p * max(1, len(terms)))()
    dtypes = (ctypes.c_int * max(1, len(terms)))()
    lds = (ctypes.c_long * max(1, len(terms)))()
    partials = (ctypes.c_int * max(1, len(terms)))()
    strides = (ctypes.c_long * max(1, len(terms)))()
    scales = (ctypes.c_float * max(1, len(terms)))()
    for i, (t, c) in enumerate(terms):
        _need_gpu(t)
        if t.dim() == 3:
            if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape[1:]) != (n_tokens, dim):
                raise KernelError(f"partial sums {tuple(t.shape)} must be contiguous float32 [P, {n_tokens}, {dim}]")
            partials[i], strides[i], lds[i] = t.shape[0], n_tokens * dim, dim
        else:
            _rows_2d(t, "an addend")
            if tuple(t.shape) != (n_tokens, dim):
                raise KernelError(f"an addend {tuple(t.shape)} does not match the residual stream {tuple(h.shape)}")
            partials[i], strides[i], lds[i] = 1, 0, (t.stride(0) if n_tokens > 1 else dim)
        ptrs[i], dtypes[i], scales[i] = t.data_ptr(), _code(t.dtype), c
    for name, t in (("weight", weight), ("bias", bias), ("weight2", weight2), ("bias2", bias2)):
        if t is not None and (t.dtype != torch.float32 or t.shape != (dim,) or not t.is_contiguous()):
            raise KernelError(f"the norm's {name} must be a contiguous float32 [{dim}] tensor")
    if (weight is None) != (bias is None) or (weight2 is None) != (bias2 is None) or (weight is None and weight2 is not None):
        raise KernelError("a layer norm has a weight and a bias; the second norm comes with a first")
    if rows is not None:
        _i32(rows, "rows")
    n_out = n_tokens if rows is None else rows.numel()
    out1 = torch.empty((n_out, dim), dtype=out_dtype, device=h.device) if weight is not None else None
    out2 = torch.empty((n_out, dim), dtype=out_dtype, device=h.device) if weight2 is not None else None
    if weight is None and not terms:
        return None
    lib = _build.load("layernorm")
    _check(
        lib,
        lib.cwm_add_layernorm(
            _ptr(h), ctypes.c_int(len(terms)), ptrs, dtypes, lds, partials, strides, scales, _ptr(weight), _ptr(bias), _ptr(out1),
            _ptr(weight2), _ptr(bias2), _ptr(out2), ctypes.c_int(_code(out_dtype)), _ptr(rows), ctypes.c_int(n_out), ctypes.c_int(dim),
            ctypes.c_float(eps), _stream(),
        ),
    )
    if weight is None:
        return None
    return out1 if weight2 is None else (out1, out2)


# --------------------------------------------------------------------------- #
MAX_MEMORY_DIM = 256  # csrc/matrix_memory.hip: MEM_MAX_DIM
MEMORY_WALK = 8  # tokens of the longest portion that a step still walks one by one; longer ones go in blocks of tokens


_MEMORY_BLOCK_TOKENS = None


def _memory_block_tokens() -> int:
    global _MEMORY_BLOCK_TOKENS
    if _MEMORY_BLOCK_TOKENS is None:
        _MEMORY_BLOCK_TOKENS = int(_build.load("matrix_memory").cwm_matrix_memory_block_tokens())
    return _MEMORY_BLOCK_TOKENS


def matrix_memory_state_elems(heads: int, dim: int, vdim: int) -> int:
    """float32 values of a request's state of `heads` matrix memories of dim x vdim, in the scan kernel's own layout:
    per head the matrix transposed, [vdim][16 * split] with split the least power of two that gives 16 * split >= dim,
    then the normaliser's 16 * split values, then the running maximum and three unused values."""
    split = 1
    while 16 * split < dim:
        split *= 2
    return heads * (vdim * 16 * split + 16 * split + 4)


def matrix_memory_state_unpack(flat: torch.Tensor, heads: int, dim: int, vdim: int):
    """(S [heads, dim, vdim], n [heads, dim], m [heads]) of one request's state row (tests read states this way)."""
    per = matrix_memory_state_elems(1, dim, vdim)
    d_pad = (per - 4) // (vdim + 1)
    rows = flat[: heads * per].reshape(heads, per)
    s = rows[:, : vdim * d_pad].reshape(heads, vdim, d_pad)[:, :, :dim].transpose(1, 2)
    return s, rows[:, vdim * d_pad : vdim * d_pad + dim], rows[:, vdim * d_pad + d_pad]


def matrix_memory(
    proj: torch.Tensor, gates: torch.Tensor, weight: torch.Tensor, state: torch.Tensor, batch: Any,
    heads: int, dim: int, vdim: int, cap: float, eps: float, q_scale: Optional[float] = None,
) -> torch.Tensor:
    """The matrix memory of `csrc/matrix_memory.hip` over the step's tokens.  `proj` [T, heads * (2 dim + 2 vdim)]
    holds, side by side, queries and keys (heads * dim each), values and the output gate's projection (heads * vdim each);
    `gates` float32 [T, 2 heads] the projections of the input gates, then of the forget gates, biases included;
    `weight` float32 [heads * vdim]; `state` float32 [slots, >= matrix_memory_state_elems], read and written at the
    sequences' slots.  Queries are multiplied by `q_scale` (default dim ** -0.5).  Returns [T, heads * vdim] in proj's
    type: every head's result over its root mean square, times weight, times sigmoid(gate).  A step whose portions all
    have up to `MEMORY_WALK` tokens (`batch.q_lens`) walks them token by token, which gives the same bits however a
    sequence is cut; a step with a longer portion takes blocks of tokens at once, which differs from the walk by rounding."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(proj, gates, weight, state)
    _rows_2d(proj, "the projection")
    _rows_2d(gates, "the gates")
    n_tokens = proj.shape[0]
    width = heads * (2 * dim + 2 * vdim)
    if proj.shape[1] != width or n_tokens != batch.n_tokens:
        raise KernelError(f"the projection {tuple(proj.shape)} must be [{batch.n_tokens}, {width}]")
    if gates.dtype != torch.float32 or tuple(gates.shape) != (n_tokens, 2 * heads):
        raise KernelError(f"the gates must be float32 [{n_tokens}, {2 * heads}]")
    if weight.dtype != torch.float32 or weight.shape != (heads * vdim,) or not weight.is_contiguous():
        raise KernelError(f"the weight must be a contiguous float32 [{heads * vdim}]")
    if dim > MAX_MEMORY_DIM:
        raise KernelError(f"heads of {dim} rows: the scan kernel takes up to {MAX_MEMORY_DIM}")
    need = matrix_memory_state_elems(heads, dim, vdim)
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] < need or not state.is_contiguous() or state.shape[1] % 4 != 0:
        raise KernelError(f"the state must be a contiguous float32 [slots, >= {need}] tensor whose rows are multiples of 16 bytes")
    coef = torch.empty((n_tokens, heads, 4), dtype=torch.float32, device=proj.device)
    y = torch.empty((n_tokens, heads * vdim), dtype=torch.float32, device=proj.device)
    out = torch.empty((n_tokens, heads * vdim), dtype=proj.dtype, device=proj.device)
    start = nq = scores = None
    q_lens = getattr(batch, "q_lens", None)
    if q_lens and max(q_lens) > MEMORY_WALK:
        start = torch.empty((batch.n_seqs, heads), dtype=torch.float64, device=proj.device)
        nq = torch.empty((n_tokens, heads), dtype=torch.float32, device=proj.device)
        scores = torch.empty((n_tokens, heads, _memory_block_tokens() + 2), dtype=torch.float32, device=proj.device)
    lib = _build.load("matrix_memory")
    _check(
        lib,
        lib.cwm_matrix_memory(
            _ptr(proj), ctypes.c_int(_code(proj.dtype)), ctypes.c_long(proj.stride(0) if n_tokens > 1 else width),
            ctypes.c_int(0), ctypes.c_int(heads * dim), ctypes.c_int(2 * heads * dim), ctypes.c_int(2 * heads * dim + heads * vdim),
            _ptr(gates), ctypes.c_long(gates.stride(0) if n_tokens > 1 else 2 * heads), ctypes.c_float(cap),
            ctypes.c_float(dim ** -0.5 if q_scale is None else q_scale), _ptr(state), ctypes.c_long(state.shape[1]), ctypes.c_int(state.shape[0]),
            _ptr(batch.cu_q), _ptr(batch.state_slots), ctypes.c_int(batch.n_seqs), ctypes.c_int(n_tokens),
            _ptr(coef), _ptr(y), _ptr(start), _ptr(nq), _ptr(scores), _ptr(weight), ctypes.c_float(eps), _ptr(out), ctypes.c_int(heads), ctypes.c_int(dim),
            ctypes.c_int(vdim), _stream(),
        ),
    )
    return out
