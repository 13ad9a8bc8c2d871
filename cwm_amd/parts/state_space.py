"""Selective state-space mixer (the Mamba-2 recurrence) with a per-request state."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import Mixer, PartChoice, Runtime, StateSpec, TensorSpec, register_part
from .linear import LinearWeights


class SelectiveStateSpace(Mixer):
    """u = W_in s = [z | x | B | C | dt] with inner = heads * head_dim channels of z and x, groups * state of B
    and C, one dt a head.  (x, B, C) pass a causal convolution per channel (`taps` wide, bias) and SiLU;
    dt <- softplus(dt + dt_bias).  Per head h with its group g = h // (heads / groups), the state S (state x
    head_dim, float32) moves as
        S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T,      y_t = S_t^T C_t + D_h x_t,
    then out = W_o norm(y * silu(z)) with a group norm of `norm_groups` parts.  The recurrence, its step sizes
    and decays and the gated norm run in float32 whatever the activation type.

    A request's state is one float32 row: S of every head (in the order the scan kernel holds it), then the last
    taps - 1 inputs of the convolution (oldest first), so a portion of a prompt goes on where the step before stopped."""

    replayable = True

    def __init__(self, dim: int, heads: int, head_dim: int, state: int, groups: int, norm_groups: int, taps: int, eps: float) -> None:
        if heads % groups != 0:
            raise ValueError(f"{heads} heads do not divide into {groups} groups")
        if not 1 <= taps <= ops.MAX_CONV_TAPS:
            raise ValueError(f"a convolution of {taps} taps is outside 1..{ops.MAX_CONV_TAPS}, what the kernel takes")
        if state > ops.MAX_SSM_STATE:
            raise ValueError(f"a state of {state} rows is more than the {ops.MAX_SSM_STATE} the scan kernel takes")
        self.dim, self.heads, self.head_dim, self.state, self.groups, self.taps = dim, heads, head_dim, state, groups, taps
        self.inner = heads * head_dim
        self.channels = self.inner + 2 * groups * state  # what the convolution sees
        self.norm = PartChoice("group_rmsnorm", {"dim": self.inner, "eps": eps, "groups": norm_groups, "tensor": "norm"}).build("norm")
        self.ssm_elems = ops.scan_state_elems(heads, head_dim, state)  # in the scan kernel's own order and padding
        self.state_elems = -(-(self.ssm_elems + (taps - 1) * self.channels) // 4) * 4

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.state_elems,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            "in": TensorSpec((2 * self.inner + 2 * self.groups * self.state + self.heads, self.dim)),
            "conv": TensorSpec((self.channels, self.taps)),
            "conv.b": TensorSpec((self.channels,)),
            "dt_bias": TensorSpec((self.heads,)),
            "A_log": TensorSpec((self.heads,)),
            "D": TensorSpec((self.heads,)),
            **self.norm.tensor_specs(),
            "o": TensorSpec((self.dim, self.inner)),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.norm.bind({"norm": tensors["norm"]}, runtime)
        self.w_in = LinearWeights(tensors["in"], stream_copy=runtime.stream_copies)
        self.w_out = LinearWeights(tensors["o"], stream_copy=runtime.stream_copies)
        # everything that enters the recurrence is kept in float32 (exact from a 16-bit file)
        self.conv_w = tensors["conv"].float().contiguous()
        self.conv_w_by_tap = self.conv_w.t().contiguous()  # [taps, channels]: what portions of a prompt read
        self.conv_b = tensors["conv.b"].float().contiguous()
        self.dt_bias = tensors["dt_bias"].float().contiguous()
        self.a_log = tensors["A_log"].float().contiguous()
        self.d_skip = tensors["D"].float().contiguous()

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        if not write_cache:
            raise ValueError("a state-space mixer cannot read another layer's state")
        u = self.w_in(x)
        inner = self.inner
        z = u[:, :inner]
        xbc = ops.causal_conv_silu(
            u[:, inner : inner + self.channels], self.conv_w, self.conv_b, cache.state, self.ssm_elems, batch, self.conv_w_by_tap,
        )
        y = ops.selective_scan(
            xbc, u[:, inner + self.channels :], self.dt_bias, self.a_log, self.d_skip, cache.state, batch,
            self.heads, self.head_dim, self.state, self.groups,
        )
        return self.w_out(self.norm.gated(y, z), partials_ok=True)


register_part("mixer", "selective_state_space", SelectiveStateSpace)


class MatrixMemory(Mixer):
    """A matrix memory per head with exponential gates and a running maximum (the mLSTM recurrence), with a
    per-request state.  q = W_q x * head_dim^(-1/2), k = W_k x (heads x head_dim), v = W_v x (heads x v_dim); per head
        i_t = c tanh((W_i x + b_i) / c),   f_t = logsigmoid(c tanh((W_f x + b_f) / c))        c = `gate_cap`
        m_t = max(f_t + m_(t-1), i_t)
        S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,      n_t the same with k_t alone
        y_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
    with S, n and m zero at a request's start; then out = W_o (y / rms(y per head) * weight * sigmoid(W_g x)).  The
    gates' projections leave their product in float32, and the gates, the maximum, the state, the result's norm and
    its gate are float32 whatever the activation type.  A request's state is one float32 row in the scan kernel's own
    layout (`ops.matrix_memory_state_elems`).  `names`: local names of the tensors for the roles q, k, v, g, o, norm,
    i, i_bias, f, f_bias."""

    replayable = True
    DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "i_bias": "i.b", "f": "f", "f_bias": "f.b"}

    def __init__(self, dim: int, heads: int, head_dim: int, v_dim: int, gate_cap: float, eps: float, names: Optional[Mapping[str, str]] = None) -> None:
        if min(heads, head_dim, v_dim) < 1 or head_dim > ops.MAX_MEMORY_DIM:
            raise ValueError(f"heads of {head_dim} x {v_dim}: the scan kernel takes 1..{ops.MAX_MEMORY_DIM} rows")
        if not gate_cap > 0:
            raise ValueError("the gates' cap must be positive")
        self.dim, self.heads, self.head_dim, self.v_dim = dim, heads, head_dim, v_dim
        self.gate_cap, self.eps = float(gate_cap), float(eps)
        self.names = {**self.DEFAULT_NAMES, **dict(names or {})}
        self.state_elems = ops.matrix_memory_state_elems(heads, head_dim, v_dim)

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.state_elems,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n = self.names
        qk, vv = self.heads * self.head_dim, self.heads * self.v_dim
        return {
            n["q"]: TensorSpec((qk, self.dim)),
            n["k"]: TensorSpec((qk, self.dim)),
            n["v"]: TensorSpec((vv, self.dim)),
            n["g"]: TensorSpec((vv, self.dim)),
            n["o"]: TensorSpec((self.dim, vv)),
            n["norm"]: TensorSpec((vv,), init="norm", precision="stored"),
            n["i"]: TensorSpec((self.heads, self.dim)),
            n["i_bias"]: TensorSpec((self.heads,), precision="stored"),
            n["f"]: TensorSpec((self.heads, self.dim)),
            n["f_bias"]: TensorSpec((self.heads,), precision="stored"),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        n = self.names
        self.proj = LinearWeights.joined([tensors[n[r]] for r in ("q", "k", "v", "g")], [None] * 4, stream_copy=runtime.stream_copies)
        self.gates = LinearWeights.joined([tensors[n["i"]], tensors[n["f"]]], [tensors[n["i_bias"]], tensors[n["f_bias"]]])
        self.w_out = LinearWeights(tensors[n["o"]], stream_copy=runtime.stream_copies)
        self.weight = tensors[n["norm"]].float().contiguous()

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        if not write_cache:
            raise ValueError("a matrix memory cannot read another layer's state")
        proj = self.proj(x)
        gates = self.gates(x, out_dtype=torch.float32)  # float32 sums, not rounded: they enter the recurrence
        y = ops.matrix_memory(proj, gates, self.weight, cache.state, batch, self.heads, self.head_dim, self.v_dim, self.gate_cap, self.eps)
        return self.w_out(y, partials_ok=True)


register_part("mixer", "matrix_memory", MatrixMemory)


class GatedLinearAttention(Mixer):
    """Linear attention with a decay per key channel, with a per-request state.  q = W_q x * head_dim^(-1/2), k = W_k x
    (heads x head_dim), v = W_v x (heads x v_dim); per head
        alpha_t = sigmoid(W_a2 (W_a1 x) + b_a)^(1 / tau)                a decay a key channel, through a low rank
        S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,      y_t = S_t^T q_t
    with S zero at a request's start; then out = W_o (y / rms(y per head) * weight * silu(W_g x)), the weight of v_dim
    values shared by the heads.  The decays' second projection leaves its product in float32, and decays, state, the
    result's norm and its gate are float32 whatever the activation type.  A request's state is one float32 row in the
    walking kernel's own layout (`ops.gla_state_elems`).  `names`: local names of the tensors for the roles q, k, v, g,
    o, norm, a1, a2, a2_bias.  `decay_rank` None: the rank is whatever the folder's a1 and a2 have (random weights are
    drawn with `DRAWN_RANK`)."""

    replayable = True
    DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a2_bias": "a2.b"}
    DRAWN_RANK = 32

    def __init__(
        self, dim: int, heads: int, head_dim: int, v_dim: int, tau: float, decay_rank: Optional[int], eps: float,
        names: Optional[Mapping[str, str]] = None,
    ) -> None:
        if min(heads, head_dim, v_dim, decay_rank or 1) < 1 or head_dim > ops.MAX_GLA_DIM:
            raise ValueError(f"heads of {head_dim} x {v_dim}: the walking kernel takes 1..{ops.MAX_GLA_DIM} rows")
        if not tau > 0:
            raise ValueError("tau must be positive")
        self.dim, self.heads, self.head_dim, self.v_dim, self.decay_rank = dim, heads, head_dim, v_dim, decay_rank
        self.tau, self.eps = float(tau), float(eps)
        self.names = {**self.DEFAULT_NAMES, **dict(names or {})}
        self._state_elems: Optional[int] = None

    @property
    def state_elems(self) -> int:
        if self._state_elems is None:
            self._state_elems = ops.gla_state_elems(self.heads, self.head_dim, self.v_dim)
        return self._state_elems

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.state_elems,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n = self.names
        qk, vv = self.heads * self.head_dim, self.heads * self.v_dim
        return {
            n["q"]: TensorSpec((qk, self.dim)),
            n["k"]: TensorSpec((qk, self.dim)),
            n["v"]: TensorSpec((vv, self.dim)),
            n["g"]: TensorSpec((vv, self.dim)),
            n["o"]: TensorSpec((self.dim, vv)),
            n["norm"]: TensorSpec((self.v_dim,), init="norm", precision="stored"),
            n["a1"]: TensorSpec((self.decay_rank or -self.DRAWN_RANK, self.dim)),
            n["a2"]: TensorSpec((qk, self.decay_rank or -self.DRAWN_RANK)),
            n["a2_bias"]: TensorSpec((qk,), precision="stored"),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        n = self.names
        if tensors[n["a1"]].shape[0] != tensors[n["a2"]].shape[1]:
            raise ValueError(f"the decays' two projections do not meet: {tuple(tensors[n['a1']].shape)} and {tuple(tensors[n['a2']].shape)}")
        self.proj = LinearWeights.joined([tensors[n[r]] for r in ("q", "k", "v", "g", "a1")], [None] * 5, stream_copy=runtime.stream_copies)
        self.width = 2 * self.heads * (self.head_dim + self.v_dim)
        self.decay_up = LinearWeights(tensors[n["a2"]], tensors[n["a2_bias"]].float())
        self.w_out = LinearWeights(tensors[n["o"]], stream_copy=runtime.stream_copies)
        self.weight = tensors[n["norm"]].float().contiguous()

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        if not write_cache:
            raise ValueError("a linear attention cannot read another layer's state")
        proj = self.proj(x)
        # the low rank's second product: exact products and float32 sums, not rounded (they enter the recurrence); its K
        # is a few tens, which the float32 kernel takes whatever the size
        logits = ops.gemm_f32(proj[:, self.width :], self.decay_up.weight, self.decay_up.bias, torch.float32)
        y = ops.gated_linear_attention(proj, logits, self.weight, cache.state, batch, self.heads, self.head_dim, self.v_dim, self.tau, self.eps)
        return self.w_out(y, partials_ok=True)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
