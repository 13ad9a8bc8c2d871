"""RMSNorm fused with the residual sum that precedes it."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import Norm, Runtime, TensorSpec, register_part


class RMSNorm(Norm):
    """y = x * rsqrt(mean(x^2) + eps) * weight, in float32
    (cwm/fastgen/kernels/rmsnorm.py:34-61; call sites cwm/fastgen/forward.py:571,
    772,789).  The residual update that the reference adds just before
    (`h.add_`, forward.py:769,786) is added here, in float32, in the same kernel."""

    replayable = True

    def __init__(self, dim: int, eps: float, offset: float = 0.0, tensor: str = "weight") -> None:
        """`offset` is added to the stored weight (1 for a weight that is stored around zero and applied as
        1 + w); `tensor` is the weight's local name ("" where the folder names it by the part's prefix alone)."""
        self.dim = dim
        self.eps = float(eps)
        self.offset = float(offset)
        self.tensor = tensor

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.dim,), init="norm" if self.offset == 0.0 else "normal", precision="stored")}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = tensors[self.tensor]
        if self.offset != 0.0:
            self.weight = (self.weight.float() + self.offset).contiguous()  # the sum in float32, once

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.add_rmsnorm(h, delta, self.weight, self.eps, self.runtime.act_dtype, rows)


register_part("norm", "rmsnorm", RMSNorm)


class GroupRMSNorm(Norm):
    """RMSNorm in `groups` equal consecutive parts: each part of a row is divided by its own
    sqrt(mean(part^2) + eps), and the whole row is multiplied by the weight; float32 arithmetic.  One group is
    the plain RMSNorm.  `tensor` is the weight's local name ("" where the folder names the weight by the part's
    prefix alone).

    Besides the norm-after-sum of `forward` it serves layers that normalise a sublayer's output before the
    residual sum (`add_normed`) and rows that are normalised where they lie (`normalize_`)."""

    replayable = True

    def __init__(self, dim: int, eps: float, groups: int = 1, tensor: str = "weight") -> None:
        if groups < 1 or dim % groups != 0:
            raise ValueError(f"{dim} elements do not divide into {groups} groups")
        self.dim = dim
        self.eps = float(eps)
        self.groups = groups
        self.tensor = tensor

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.dim,), init="norm", precision="stored")}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = tensors[self.tensor].contiguous()

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        if delta is not None:
            if rows is not None:
                raise ValueError("a pending residual update with a choice of rows is not served by the group norm")
            ops.add_rows(h, delta)
        return ops.group_rmsnorm(h, self.weight, self.groups, self.eps, self.runtime.act_dtype, rows=rows)

    def add_normed(self, h: torch.Tensor, y: torch.Tensor, also: Optional[torch.dtype] = None) -> Optional[torch.Tensor]:
        """h (float32 [T, D]) += norm(y) * weight; `y` is [T, D] or float32 partial sums [P, T, D].  With `also` the
        rows of h as they then stand are returned in that type as well (h itself if it is float32): what the next
        sublayer reads, from the same kernel."""
        copy = None
        if also is not None and also != h.dtype:
            copy = torch.empty(h.shape, dtype=also, device=h.device)
        ops.group_rmsnorm(y, self.weight, self.groups, self.eps, torch.float32, out=h, accumulate=True, copy=copy)
        return copy if copy is not None else (h if also is not None else None)

    def normalize_(self, x: torch.Tensor) -> torch.Tensor:
        """Rows of `x` ([T, D], the rows may lie apart) normalised in place."""
        return ops.group_rmsnorm(x, self.weight, self.groups, self.eps, x.dtype, out=x)

    def gated(self, y: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
        """norm(y * silu(gate)) * weight in the activation type: the gate is applied before the norm."""
        return ops.group_rmsnorm(y, self.weight, self.groups, self.eps, self.runtime.act_dtype, gate=gate)


register_part("norm", "group_rmsnorm", GroupRMSNorm)


@dataclass
class StreamUpdate:
    """A sublayer's result that has not yet gone into a residual of several streams: `y` ([T, D], float32 partial
    sums [P, T, D], or an `ops.RoutedSum`) with the coefficients that take it there, x_t <- sum_s mix[s, t] x_s + out_coef[t] y (float32
    [S, S] and [S]; None for the identity and ones, which is the plain residual sum)."""

    y: Any
    mix: Optional[torch.Tensor] = None
    out_coef: Optional[torch.Tensor] = None


class StreamRMSNorm(RMSNorm):
    """RMSNorm of what a sublayer reads from a residual of `streams` vectors a token (float32 [T, streams * D]):
    u = sum_s in_coef[s] x_s, then u / sqrt(mean(u^2) + eps) * (offset + weight).  The pending `StreamUpdate` of the
    sublayer before is applied to the streams first, in the same kernel and in float32.  Without `in_coef` every
    stream counts once: the sum of the streams, which is what a model's final norm reads.  One stream with no
    coefficients is the ordinary residual."""

    def __init__(self, dim: int, eps: float, streams: int = 1, offset: float = 0.0, tensor: str = "weight") -> None:
        super().__init__(dim, eps, offset, tensor)
        if not 1 <= streams <= ops.MAX_STREAMS:
            raise ValueError(f"{streams} streams: the kernels take 1..{ops.MAX_STREAMS}")
        self.streams = streams

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = self.weight.float().contiguous()

    def forward(  # type: ignore[override]
        self, h: torch.Tensor, delta: Optional[StreamUpdate], rows: Optional[torch.Tensor] = None, in_coef: Optional[torch.Tensor] = None,
    ) -> torch.Tensor:
        y, mix, out_coef = (delta.y, delta.mix, delta.out_coef) if delta is not None else (None, None, None)
        return ops.stream_mix_norm(h, self.streams, y, mix, out_coef, in_coef, self.weight, self.eps, self.runtime.act_dtype, rows)


register_part("norm", "stream_rmsnorm", StreamRMSNorm)


class LayerNorm(Norm):
    """y = (x - mean(x)) / sqrt(var(x) + eps) * weight + bias, the variance being the mean squared deviation; float32
    arithmetic.  The pending residual update is added first, in the same kernel and in float32; it may be a tensor,
    partial sums, or an `ops.ScaledSum` of several sublayers' results.  `tensor` and `bias_tensor` are the local names
    of weight and bias.  `forward_pair` serves layers whose sublayers read the same residual through norms of their
    own: both norms share the mean and the variance, and one kernel writes both."""

    replayable = True

    def __init__(self, dim: int, eps: float, tensor: str = "weight", bias_tensor: str = "bias") -> None:
        self.dim = dim
        self.eps = float(eps)
        self.tensor = tensor
        self.bias_tensor = bias_tensor

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            self.tensor: TensorSpec((self.dim,), init="norm", precision="stored"),
            self.bias_tensor: TensorSpec((self.dim,), init="normal", precision="stored"),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weight = tensors[self.tensor].float().contiguous()
        self.bias = tensors[self.bias_tensor].float().contiguous()

    def forward(self, h: torch.Tensor, delta: Any, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.add_layernorm(h, delta, self.weight, self.bias, self.eps, self.runtime.act_dtype, rows)

    def forward_pair(self, h: torch.Tensor, delta: Any, other: "LayerNorm"):
        """This norm's rows and `other`'s, of the same residual after the same update."""
        if other.dim != self.dim or other.eps != self.eps:
            raise ValueError("two norms share their statistics only with one size and one eps")
        return ops.add_layernorm(h, delta, self.weight, self.bias, self.eps, self.runtime.act_dtype, None, other.weight, other.bias)


register_part("norm", "layernorm", LayerNorm)
