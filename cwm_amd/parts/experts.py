"""Routed experts: a feed-forward of which each token uses a few."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import FeedForward, PartChoice, Runtime, TensorSpec, register_part


class RoutedExperts(FeedForward):
    """z = W_router x in float32; a token's `top` experts are those with the largest z, weighted by the softmax
    over these z alone; out = sum_e weight_e * W_down,e (silu(W_gate,e x) * (W_up,e x)), no biases.

    Other routers and experts by argument.  `scores` "softmax_all": s = softmax(z) over all experts; the `top`
    experts with the largest s + correction (tensor `correction` [experts], if `correction`) are chosen and weighted
    by `weight_scale` * s, the correction not included, divided by the chosen scores' sum first if `renormalize`.
    `activation` "clamped_swish": an expert makes g' * sigmoid(act_alpha * g') * (u' + 1) of g = W_gate x and
    u = W_up x, with g' = min(g, act_limit) and u' = clamp(u, -act_limit, act_limit).

    The step's (token, expert) pairs are grouped by expert on the device (no count comes to the host), each
    group's rows padded to whole tiles, and two grouped products run over the tiles: gate/up with the
    activation in its epilogue, then down into one float32 row a pair; a last kernel adds a token's rows in the
    order of its router's choice, so a token's result does not depend on what else is in the step.
    With `router_bias` the logits are W_router x + b (tensor `router.b`).  `shared`: a feed-forward of the registry that
    runs for every token beside the chosen experts (its tensors under `shared_prefix`); `forward` then returns the
    two results as an `ops.ScaledSum`, which whoever adds the layer's results into the residual adds up.
    Tensors: `router` [experts, dim] and `e<i>.gate`, `e<i>.up` [hidden, dim], `e<i>.down` [dim, hidden]."""

    replayable = True

    def __init__(
        self, dim: int, hidden_dim: int, n_experts: int, top: int, scores: str = "softmax_chosen", correction: bool = False,
        weight_scale: float = 1.0, renormalize: bool = False, activation: str = "silu", act_alpha: float = 1.0, act_limit: float = 0.0,
        router_bias: bool = False, shared: Optional[PartChoice] = None, shared_prefix: str = "shared.",
    ) -> None:
        if not 1 <= top <= n_experts:
            raise ValueError(f"{top} experts a token out of {n_experts}")
        if top > ops.MAX_ROUTE_TOP or n_experts > ops.MAX_EXPERTS:
            raise ValueError(f"the routing kernels take up to {ops.MAX_ROUTE_TOP} of up to {ops.MAX_EXPERTS} experts")
        if scores not in ("softmax_chosen", "softmax_all"):
            raise ValueError(f"router scores {scores!r}: 'softmax_chosen' and 'softmax_all' are known")
        if scores == "softmax_chosen" and (correction or weight_scale != 1.0 or renormalize):
            raise ValueError("a correction, a scale and renormalised weights belong to router scores over all experts")
        self.dim, self.hidden_dim, self.n_experts, self.top = dim, hidden_dim, n_experts, top
        self.scores, self.correction, self.weight_scale, self.renormalize = scores, correction, float(weight_scale), renormalize
        self.activation = ops.GatedActivation(activation, float(act_alpha), float(act_limit))
        self.activation.code()  # an unknown kind is refused here
        self.router_bias = router_bias
        self.shared: Optional[FeedForward] = shared.build("feed_forward") if shared is not None else None  # type: ignore[assignment]
        self.shared_prefix = shared_prefix

    @property
    def replayable(self) -> bool:  # type: ignore[override]
        return self.shared is None or self.shared.replayable

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {"router": TensorSpec((self.n_experts, self.dim))}
        if self.router_bias:
            specs["router.b"] = TensorSpec((self.n_experts,), precision="stored")
        if self.shared is not None:
            specs.update({self.shared_prefix + name: spec for name, spec in self.shared.tensor_specs().items()})
        if self.correction:
            specs["correction"] = TensorSpec((self.n_experts,), init="zeros", precision="stored")
        for e in range(self.n_experts):
            specs[f"e{e}.gate"] = TensorSpec((self.hidden_dim, self.dim))
            specs[f"e{e}.up"] = TensorSpec((self.hidden_dim, self.dim))
            specs[f"e{e}.down"] = TensorSpec((self.dim, self.hidden_dim))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.router = tensors["router"].contiguous()
        self.router_b = tensors["router.b"].float().contiguous() if self.router_bias else None
        if self.shared is not None:
            n = len(self.shared_prefix)
            self.shared.bind({name[n:]: t for name, t in tensors.items() if name.startswith(self.shared_prefix)}, runtime)
        self.choice_correction = tensors["correction"].float().contiguous() if self.correction else None
        stack = lambda name: torch.stack([tensors[f"e{e}.{name}"] for e in range(self.n_experts)]).contiguous()  # noqa: E731
        self.gate, self.up, self.down = stack("gate"), stack("up"), stack("down")  # [experts, out, in]

    def forward(self, x: torch.Tensor, batch: Any) -> Any:
        routed = self.forward_deferred(x, batch).combine()  # float32 [T, dim]
        if self.shared is None:
            return routed
        return ops.ScaledSum([(routed, 1.0), (self.shared.forward(x, batch), 1.0)])

    def forward_deferred(self, x: torch.Tensor, batch: Any) -> "ops.RoutedSum":
        """The same without the last kernel: every pair's row and the weights, for a consumer that adds a token's
        rows up itself (a norm that takes a `RoutedSum` as the pending result)."""
        logits = ops.linear(x, self.router, self.router_b, torch.float32)
        chosen, weights = ops.route_top(logits, self.top, self.scores, self.choice_correction, self.weight_scale, self.renormalize)
        groups = ops.group_by_expert(chosen, self.n_experts)
        if self.activation.kind == "silu":
            hidden = ops.grouped_gate_up(x, groups, self.gate, self.up)
        else:
            hidden = ops.grouped_gate_up(x, groups, self.gate, self.up, self.activation)
        rows = ops.grouped_linear(hidden, groups, self.down)
        return ops.RoutedSum(rows, groups, weights)


register_part("feed_forward", "routed_experts", RoutedExperts)
