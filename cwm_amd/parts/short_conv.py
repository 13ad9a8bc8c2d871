"""Short causal convolutions on what a layer's sublayers read."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional, Sequence, Tuple

import torch

from .. import ops
from .base import Mixer, Runtime, StateSpec, TensorSpec, register_part


class InputConvolution(Mixer):
    """What each of a layer's sublayers reads in place of the normalised rows h: h + conv(h), a causal convolution over
    time on each channel with weights of the sublayer's own,
        conv(h)_t = sum_(lag = 0 .. taps - 1) w[:, taps - 1 - lag] * h_(t - lag),     h_t = 0 for t < 0, no bias.
    `outputs` names the weights' tensors, one a sublayer ([dim, taps] each); `forward` returns as many tensors.  All
    of them read the same h, so the last taps - 1 rows of h are one state of the sequence (float32 [(taps - 1) * dim],
    oldest first): a mixer with a state of its own, like a token shift.  `ignored` names weights of sublayers that the
    layer does not have: a folder may hold them, nothing reads them.  float32 arithmetic."""

    replayable = True

    def __init__(self, dim: int, taps: int, outputs: Sequence[str] = ("weight",), ignored: Sequence[str] = ()) -> None:
        if not 1 <= taps <= ops.MAX_SHORT_CONV_TAPS:
            raise ValueError(f"a convolution of {taps} taps is outside 1..{ops.MAX_SHORT_CONV_TAPS}, what the kernel takes")
        if not 1 <= len(outputs) <= 2:
            raise ValueError("one or two convolutions of the same input are taken")
        self.dim, self.taps, self.outputs, self.ignored = dim, taps, tuple(outputs), tuple(ignored)

    def cache_spec(self) -> Optional[StateSpec]:
        if self.taps == 1:
            return None  # the current token's tap alone: nothing is carried
        return StateSpec(((self.taps - 1) * self.dim,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {name: TensorSpec((self.dim, self.taps)) for name in self.outputs}
        specs.update({name: TensorSpec((self.dim, self.taps), optional=True) for name in self.ignored})
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        # a row a tap, in float32 (exact from a 16-bit file): what the kernel reads channel by channel
        self.by_tap = [tensors[name].float().t().contiguous() for name in self.outputs]

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> Tuple[torch.Tensor, ...]:
        return ops.short_conv(x, self.by_tap, cache.state if cache is not None else None, batch, write_state=write_cache)


register_part("mixer", "input_convolution", InputConvolution)
