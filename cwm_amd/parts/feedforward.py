"""Dense feed-forwards: gated, and with a plain activation between two products."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import FeedForward, Runtime, TensorSpec, register_part
from .linear import LinearWeights


class SwiGLU(FeedForward):
    """w2(silu(w1 x) * (w3 x)), no biases (cwm/fastgen/forward.py:776-782;
    cwm/model/transformer.py:214-228).  w1 and w3 are joined into one product; the
    gate's SiLU and the product with the up branch are computed in float32 and
    rounded once."""

    replayable = True

    def __init__(self, dim: int, hidden_dim: int) -> None:
        self.dim = dim
        self.hidden_dim = hidden_dim

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            "w1.weight": TensorSpec((self.hidden_dim, self.dim)),
            "w2.weight": TensorSpec((self.dim, self.hidden_dim)),
            "w3.weight": TensorSpec((self.hidden_dim, self.dim)),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        # gate and up rows alternate in groups of 8 where the width allows, so that a decode batch
        # finishes silu(gate) * up in the product's epilogue
        self.grouped = self.hidden_dim % 8 == 0
        self.gate_up = LinearWeights.joined(
            [tensors["w1.weight"], tensors["w3.weight"]], [None, None], group=8 if self.grouped else None,
            stream_copy=runtime.stream_copies,
        )
        self.down = LinearWeights(tensors["w2.weight"], stream_copy=runtime.stream_copies)

    def forward(self, x: torch.Tensor, batch: Any) -> torch.Tensor:
        # the result (or partial sums of it) is added into the residual by the next norm.  (Forming
        # silu(gate) * up inside the down product was tried: every block recomputes it, which costs
        # more than the kernel it saves.)
        hidden = ops.gate_up_silu(x, self.gate_up.weight, self.gate_up.bias, self.grouped, streamed=self.gate_up.streamed)
        return self.down(hidden, partials_ok=True)


register_part("feed_forward", "swiglu", SwiGLU)


class ActivatedMLP(FeedForward):
    """W_down act(W_up x), no gate and no biases; `activation` is one of `ops.ACTIVATIONS` ("relu2": the square of
    relu).  The activation is computed in float32 on the product's sums and rounded once.  `up` and `down` are
    the tensors' local names."""

    replayable = True

    def __init__(self, dim: int, hidden_dim: int, activation: str = "relu2", up: str = "up", down: str = "down") -> None:
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"activation {activation!r}: known are {', '.join(ops.ACTIVATIONS)}")
        self.dim, self.hidden_dim, self.activation = dim, hidden_dim, activation
        self.up_name, self.down_name = up, down

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.up_name: TensorSpec((self.hidden_dim, self.dim)), self.down_name: TensorSpec((self.dim, self.hidden_dim))}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.up = LinearWeights(tensors[self.up_name], stream_copy=runtime.stream_copies)
        self.down = LinearWeights(tensors[self.down_name], stream_copy=runtime.stream_copies)

    def forward(self, x: torch.Tensor, batch: Any) -> torch.Tensor:
        hidden = ops.act_rows(self.up(x, partials_ok=True), self.activation, x.dtype)
        return self.down(hidden, partials_ok=True)


register_part("feed_forward", "activated_mlp", ActivatedMLP)


class GatedMLP(FeedForward):
    """W_down act(W_gate x, W_up x), no biases, with the gated activation as an argument (`ops.GatedActivation`):
    "silu": silu(g) * u;  "clamped_swish": g' * sigmoid(act_alpha * g') * (u' + 1) with g' = min(g, act_limit) and
    u' = clamp(u, -act_limit, act_limit).  With `row_gate` (a tensor's local name, [1, dim]) the whole result is
    multiplied by sigmoid(w . x), one number a token: the gate's row rides as one more output of the joined gate/up
    product and scales the activation's rows, which the linear down product carries through.  The activation is
    computed in float32 on the product's sums and rounded once.  `gate`, `up`, `down`: the tensors' local names."""

    replayable = True

    def __init__(
        self, dim: int, hidden_dim: int, activation: str = "silu", act_alpha: float = 1.0, act_limit: float = 0.0,
        row_gate: Optional[str] = None, gate: str = "gate", up: str = "up", down: str = "down",
    ) -> None:
        self.dim, self.hidden_dim = dim, hidden_dim
        self.activation = ops.GatedActivation(activation, float(act_alpha), float(act_limit))
        self.activation.code()  # an unknown kind is refused here
        self.row_gate, self.gate_name, self.up_name, self.down_name = row_gate, gate, up, down

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {
            self.gate_name: TensorSpec((self.hidden_dim, self.dim)),
            self.up_name: TensorSpec((self.hidden_dim, self.dim)),
            self.down_name: TensorSpec((self.dim, self.hidden_dim)),
        }
        if self.row_gate is not None:
            specs[self.row_gate] = TensorSpec((1, self.dim))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        matrices = [tensors[self.gate_name], tensors[self.up_name]]
        if self.row_gate is not None:
            matrices.append(tensors[self.row_gate])
        self.gate_up = LinearWeights.joined(matrices, [None] * len(matrices), stream_copy=runtime.stream_copies)
        self.down = LinearWeights(tensors[self.down_name], stream_copy=runtime.stream_copies)

    def forward(self, x: torch.Tensor, batch: Any) -> torch.Tensor:
        joined = self.gate_up(x, partials_ok=True)
        hidden = ops.gated_act_rows(joined, self.hidden_dim, self.activation, x.dtype, 2 * self.hidden_dim if self.row_gate is not None else None)
        return self.down(hidden, partials_ok=True)


register_part("feed_forward", "gated_mlp", GatedMLP)
