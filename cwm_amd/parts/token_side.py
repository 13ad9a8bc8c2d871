"""A layer's own input from the step's tokens."""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from .. import ops
from .base import Runtime, TensorSpec, TokenInput, register_part


class GatedTokenSide(TokenInput):
    """Every token has a second embedding row, `table` [vocab, layers * side_dim], of which the layer with index
    `index` reads the columns [index * side_dim, (index + 1) * side_dim), e.  With x the residual after the layer's
    sublayers:
        g = gelu_tanh(W_gate x) * e;   y = W_proj g;   x <- x + y / sqrt(mean(y^2) + eps) * n
    (W_gate [side_dim, dim], W_proj [dim, side_dim], n [dim]: a plain weight).  The table is one tensor of the model
    that every layer's part names (`table`, a full name of the folder); `gate`, `proj`, `norm` are the local names of
    the layer's own tensors.  Sums, activation and norm are float32; x and g enter the products rounded to the
    activation type."""

    replayable = True
    adds_pending = True  # `forward` also does the residual sum that is still pending, in the same kernel

    def __init__(
        self, vocab_size: int, dim: int, side_dim: int, index: int, n_parts: int, eps: float,
        table: str = "/side.embed", gate: str = "gate", proj: str = "proj", norm: str = "norm",
    ) -> None:
        if not 0 <= index < n_parts:
            raise ValueError(f"part {index} of a table of {n_parts} parts")
        if not 1 <= side_dim <= ops.MAX_SIDE_DIM:
            raise ValueError(f"{side_dim} side values are outside 1..{ops.MAX_SIDE_DIM}, what the kernel takes")
        if not table.startswith("/"):
            raise ValueError("the table is shared between layers: its name is a full name of the folder, with a leading '/'")
        self.vocab_size, self.dim, self.side_dim, self.index, self.n_parts, self.eps = vocab_size, dim, side_dim, index, n_parts, float(eps)
        self.table_name, self.gate_name, self.proj_name, self.norm_name = table, gate, proj, norm

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            self.table_name: TensorSpec((self.vocab_size, self.n_parts * self.side_dim)),
            self.gate_name: TensorSpec((self.side_dim, self.dim)),
            self.proj_name: TensorSpec((self.dim, self.side_dim)),
            self.norm_name: TensorSpec((self.dim,), init="norm", precision="stored"),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.table = tensors[self.table_name]
        self.w_gate = tensors[self.gate_name].contiguous()
        self.w_proj_t = tensors[self.proj_name].t().contiguous()  # a row a side value: what the kernel reads along the width
        self.weight = tensors[self.norm_name].float().contiguous()

    def forward(self, h: torch.Tensor, batch: Any, pending: Any = None) -> None:
        ops.token_side(
            h, batch.tokens, self.table, self.index * self.side_dim, self.w_gate, self.w_proj_t, self.weight, self.eps,
            round_inputs=self.runtime.act_dtype == torch.bfloat16, pending=pending,
        )


register_part("token_input", "gated_token_side", GatedTokenSide)
