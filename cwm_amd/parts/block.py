"""Arrangements of parts in one layer."""

from __future__ import annotations

from typing import Any, Mapping, Optional

import torch

from .base import Block, Connection, FeedForward, Mixer, Norm, TokenInput, register_part


class PreNormBlock(Block):
    """h += mixer(norm1(h)); h += feed_forward(norm2(h))  (cwm/fastgen/forward.py:563-786).

    Each residual sum is done by the norm that follows it, in float32: the block
    takes the previous layer's pending update and returns its own.
    """

    def __init__(self, names: Mapping[str, str], norm1: Norm, mixer: Mixer, norm2: Norm, feed_forward: FeedForward) -> None:
        super().__init__(names, norm1=norm1, mixer=mixer, norm2=norm2, feed_forward=feed_forward)
        self.norm1 = norm1
        self.mixer = mixer
        self.norm2 = norm2
        self.feed_forward = feed_forward

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        x = self.norm1.forward(h, delta)
        mixed = self.mixer.forward(x, batch, cache, write_cache)
        x = self.norm2.forward(h, mixed)
        return self.feed_forward.forward(x, batch)


register_part("block", "pre_norm", PreNormBlock)


class PostNormBlock(Block):
    """h += norm1(mixer(s)); h += norm2(feed_forward(h)): each sublayer reads the residual stream itself and its
    output is normalised before it joins the stream.  What the mixer reads, s, is the stream after the block's
    `shift` (a mixer of its own with its own state, a token shift for instance), or the stream itself in the
    activation type where the layer has none.  A layer without a feed-forward names neither `feed_forward`
    nor `norm2`.  The norms add into the stream themselves (`add_normed`), so the block leaves no pending update."""

    def __init__(
        self, names: Mapping[str, str], mixer: Mixer, norm1: Norm, shift: Optional[Mixer] = None,
        feed_forward: Optional[FeedForward] = None, norm2: Optional[Norm] = None,
    ) -> None:
        if (feed_forward is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        parts = {}
        if shift is not None:
            parts["shift"] = shift
        parts.update(mixer=mixer, norm1=norm1)
        if feed_forward is not None:
            parts.update(feed_forward=feed_forward, norm2=norm2)
        super().__init__(names, **parts)
        self.shift, self.mixer, self.norm1, self.feed_forward, self.norm2 = shift, mixer, norm1, feed_forward, norm2

    def forward(self, h: torch.Tensor, delta: Optional[torch.Tensor], batch: Any, cache: Any, write_cache: bool = True) -> None:
        from .. import ops

        if delta is not None:
            ops.add_rows(h, delta)
        act = self.runtime.act_dtype
        if self.shift is not None:
            shift_cache, mixer_cache = cache
            s = self.shift.forward(h, batch, shift_cache, write_cache)
        else:
            mixer_cache = cache
            s = ops.cast_rows(h, act)
        mixed = self.mixer.forward(s, batch, mixer_cache, write_cache)
        if self.feed_forward is None:
            self.norm1.add_normed(h, mixed)
        else:
            x = self.norm1.add_normed(h, mixed, also=act)  # the stream after the sum, as the feed-forward reads it
            self.norm2.add_normed(h, self.feed_forward.forward(x, batch))
        return None


register_part("block", "post_norm", PostNormBlock)


class ConnectedPreNormBlock(Block):
    """Pre-norm sublayers joined to the residual by connections of their own: the mixer reads
    norm1(connection1's view of the residual) and its result goes back through connection1, then the same for the
    feed-forward with norm2 and connection2 where the layer has one.  The residual may be several streams
    (`HyperConnection`) or one (`ResidualSum`); the norms (`StreamRMSNorm`) apply the pending change of the sublayer
    before and read the streams in one kernel, so the block takes the previous layer's pending change and returns
    its own, like `PreNormBlock`."""

    def __init__(
        self, names: Mapping[str, str], norm1: Norm, connection1: Connection, mixer: Mixer,
        norm2: Optional[Norm] = None, connection2: Optional[Connection] = None, feed_forward: Optional[FeedForward] = None,
    ) -> None:
        if not ((feed_forward is None) == (norm2 is None) == (connection2 is None)):
            raise ValueError("a feed-forward comes with its norm and its connection")
        parts = dict(norm1=norm1, connection1=connection1, mixer=mixer)
        if feed_forward is not None:
            parts.update(norm2=norm2, connection2=connection2, feed_forward=feed_forward)
        super().__init__(names, **parts)
        self.norm1, self.connection1, self.mixer = norm1, connection1, mixer
        self.norm2, self.connection2, self.feed_forward = norm2, connection2, feed_forward

    def forward(self, h: torch.Tensor, delta: Any, batch: Any, cache: Any, write_cache: bool = True) -> Any:
        x = self.norm1.forward(h, delta, in_coef=self.connection1.in_coef())
        delta = self.connection1.update(self.mixer.forward(x, batch, cache, write_cache))
        if self.feed_forward is not None:
            x = self.norm2.forward(h, delta, in_coef=self.connection2.in_coef())
            # a feed-forward whose result is a weighted sum of rows leaves the sum to the norm that reads it next
            deferred = getattr(self.feed_forward, "forward_deferred", None)
            delta = self.connection2.update(deferred(x, batch) if deferred is not None else self.feed_forward.forward(x, batch))
        return delta


register_part("block", "connected_pre_norm", ConnectedPreNormBlock)


class ParallelPreNormBlock(Block):
    """h += mixer(norm1(h)) + feed_forward(norm2(h)): both sublayers read the same residual, each through a norm of
    its own, and their results join it in one sum.  The sum is left to the norm that reads the residual next (an
    `ops.ScaledSum` of the sublayers' results, added in float32), and where the two norms can share their statistics
    (`forward_pair`) one kernel makes both sublayers' inputs.  A mixer that is several side by side (it lists them
    as `children()`) gets a cache slot for each child; a layer without a feed-forward names neither `feed_forward`
    nor `norm2`."""

    def __init__(
        self, names: Mapping[str, str], norm1: Norm, mixer: Mixer, norm2: Optional[Norm] = None, feed_forward: Optional[FeedForward] = None,
    ) -> None:
        if (feed_forward is None) != (norm2 is None):
            raise ValueError("a feed-forward and its norm come together")
        parts = dict(norm1=norm1, mixer=mixer)
        if feed_forward is not None:
            parts.update(norm2=norm2, feed_forward=feed_forward)
        super().__init__(names, **parts)
        self.norm1, self.mixer, self.norm2, self.feed_forward = norm1, mixer, norm2, feed_forward

    def mixers(self):
        children = getattr(self.mixer, "children", None)
        return list(children()) if children is not None else [self.mixer]

    def forward(self, h: torch.Tensor, delta: Any, batch: Any, cache: Any, write_cache: bool = True) -> Any:
        from .. import ops

        if self.feed_forward is None:
            x1, x2 = self.norm1.forward(h, delta), None
        elif hasattr(self.norm1, "forward_pair"):
            x1, x2 = self.norm1.forward_pair(h, delta, self.norm2)
        else:
            x1 = self.norm1.forward(h, delta)
            x2 = self.norm2.forward(h, None)
        mixed = self.mixer.forward(x1, batch, cache, write_cache)
        terms = list(mixed.terms) if isinstance(mixed, ops.ScaledSum) else [(mixed, 1.0)]
        if self.feed_forward is not None:
            terms.append((self.feed_forward.forward(x2, batch), 1.0))
        return ops.ScaledSum(terms)


register_part("block", "parallel_pre_norm", ParallelPreNormBlock)


class SharedNormParallelBlock(Block):
    """h += mixer(u_1) + feed_forward(u_2), where both sublayers read one norm of the residual, n = norm(h): u_1 = u_2 = n,
    or, with `conv` (a mixer with a state of its own that makes one input a sublayer from n: short convolutions over
    time), u_1, u_2 = conv(n).  With `token_input` the layer then adds its own input from the step's tokens, which
    reads the residual after the sublayers' sum: that sum is then done here (float32, the sublayers' results in their
    order; by the token input's own kernel where it says `adds_pending`) and the block leaves no pending update; without one the sum is left to the norm that
    reads the residual next, as in `ParallelPreNormBlock`.  A layer without a feed-forward names none.

    The block's mixers, in the order of their caches: `conv` where there is one, then the mixer (or its children).
    A run-order entry may let the mixer read another entry's cache while the convolution keeps a state of its own:
    `write_cache` is then a tuple, one boolean a mixer."""

    def __init__(
        self, names: Mapping[str, str], norm: Norm, mixer: Mixer, conv: Optional[Mixer] = None,
        feed_forward: Optional[FeedForward] = None, token_input: Optional[TokenInput] = None,
    ) -> None:
        parts = dict(norm=norm)
        if conv is not None:
            parts["conv"] = conv
        parts["mixer"] = mixer
        if feed_forward is not None:
            parts["feed_forward"] = feed_forward
        if token_input is not None:
            parts["token_input"] = token_input
        super().__init__(names, **parts)
        self.norm, self.conv, self.mixer, self.feed_forward, self.token_input = norm, conv, mixer, feed_forward, token_input

    def mixers(self):
        children = getattr(self.mixer, "children", None)
        own = list(children()) if children is not None else [self.mixer]
        return ([self.conv] if self.conv is not None else []) + own

    def forward(self, h: torch.Tensor, delta: Any, batch: Any, cache: Any, write_cache: Any = True) -> Any:
        from .. import ops

        views = cache if isinstance(cache, tuple) else ((cache,) if len(self.mixers()) == 1 else ())
        writes = tuple(write_cache) if isinstance(write_cache, tuple) else (write_cache,) * len(views)
        x = self.norm.forward(h, delta)
        x1 = x2 = x
        if self.conv is not None:
            made = self.conv.forward(x, batch, views[0], writes[0])
            x1, x2 = made[0], made[-1]
            views, writes = views[1:], writes[1:]
        if len(set(writes)) > 1:
            raise ValueError("the mixers side by side of one layer all write their caches or all read another layer's")
        mixed = self.mixer.forward(x1, batch, views[0] if len(views) == 1 else views, writes[0])
        terms = list(mixed.terms) if isinstance(mixed, ops.ScaledSum) else [(mixed, 1.0)]
        if self.feed_forward is not None:
            out = self.feed_forward.forward(x2, batch)
            terms.extend(out.terms if isinstance(out, ops.ScaledSum) else [(out, 1.0)])
        if self.token_input is None:
            return ops.ScaledSum(terms)
        if self.token_input.adds_pending and len(terms) <= ops.MAX_SIDE_ADDENDS:
            self.token_input.forward(h, batch, pending=ops.ScaledSum(terms))  # the sum in the input's own kernel
        else:
            ops.add_layernorm(h, ops.ScaledSum(terms), None, None, 1.0, self.runtime.act_dtype)  # the sum alone
            self.token_input.forward(h, batch)
        return None


register_part("block", "shared_norm_parallel", SharedNormParallelBlock)
