"""Causal grouped-query attention over a paged cache."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import ChunkedKVSpec, Mixer, PagedKVSpec, PartChoice, PositionEncoding, Runtime, TensorSpec, register_part
from .linear import LinearWeights


MAX_HEAD_DIM = 256  # the attention kernels' largest head size (csrc/attention_simple.hip, attention_mfma.hip)


class PagedAttention(Mixer):
    """x -> wo(attention(rope(wq x), cache of rope(wk x), cache of wv x)).

    cwm/fastgen/forward.py:593-656,763: three projections of the same input, heads
    as the slow axis of the projected features, rotation of queries and keys,
    cache write before the attention, softmax(q k^T * scale) v over the sequence's
    cached keys up to the query's own position (and no further back than the
    window), query head h reading key/value head h // (n_heads / n_kv_heads), and
    the output projection.  Every constant is an argument: sizes, `scale`
    (the reference fixes head_dim ** -0.5 at forward.py:651), `window` (keys read
    per query, own included; None for all), `bias` on the three input projections
    (cwm/model/transformer.py:173-187) and the position encoding.
    """

    def __init__(
        self,
        dim: int,
        n_heads: int,
        n_kv_heads: int,
        head_dim: int,
        scale: float,
        window: Optional[int] = None,
        bias: bool = False,
        position_encoding: Optional[PartChoice] = None,
    ) -> None:
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"{n_heads} query heads do not divide into {n_kv_heads} key/value heads")
        if not 1 <= head_dim <= MAX_HEAD_DIM:
            raise ValueError(f"head_dim {head_dim} is outside 1..{MAX_HEAD_DIM}, the sizes the attention kernels take")
        self.dim = dim
        self.n_heads = n_heads
        self.n_kv_heads = n_kv_heads
        self.head_dim = head_dim
        self.scale = float(scale)
        self.window = window
        self.bias = bias
        self.position_encoding: Optional[PositionEncoding] = (
            position_encoding.build("position_encoding") if position_encoding is not None else None
        )

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, window=self.window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        q_out = self.n_heads * self.head_dim
        kv_out = self.n_kv_heads * self.head_dim
        specs = {
            "wq.weight": TensorSpec((q_out, self.dim)),
            "wk.weight": TensorSpec((kv_out, self.dim)),
            "wv.weight": TensorSpec((kv_out, self.dim)),
            "wo.weight": TensorSpec((self.dim, q_out)),
        }
        if self.bias:
            specs["wq.bias"] = TensorSpec((q_out,))
            specs["wk.bias"] = TensorSpec((kv_out,))
            specs["wv.bias"] = TensorSpec((kv_out,))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        if self.position_encoding is not None:
            self.position_encoding.bind({}, runtime)
        names = ("wq", "wk", "wv")
        weights = {n: tensors[f"{n}.weight"] for n in names}
        biases = {n: tensors.get(f"{n}.bias") for n in names}
        pairing = self.position_encoding.rotary_pairing() if self.position_encoding is not None else "adjacent"
        # element j of a head as `transform_qk` sees it is element qk_order[j] of the head as the folder's wq and wk give it
        self.qk_order = torch.arange(self.head_dim)
        if pairing == "halves":
            # the kernels turn adjacent elements: bring element i and i + head_dim / 2 of every query and key
            # head side by side, once, by the order of the projections' rows
            half = self.head_dim // 2
            order = torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1)
            self.qk_order = order
            for n, heads in (("wq", self.n_heads), ("wk", self.n_kv_heads)):
                rows = (torch.arange(heads)[:, None] * self.head_dim + order[None, :]).reshape(-1).to(weights[n].device)
                weights[n] = weights[n][rows]
                if biases[n] is not None:
                    biases[n] = biases[n][rows]
        elif pairing != "adjacent":
            raise ValueError(f"rotary pairing {pairing!r}: 'adjacent' and 'halves' are known")
        self.qkv = LinearWeights.joined([weights[n] for n in names], [biases[n] for n in names], stream_copy=runtime.stream_copies)
        self.wo = LinearWeights(tensors["wo.weight"], stream_copy=runtime.stream_copies)
        # a subclass that changes queries and keys between projection and rotation cannot use the fused product
        self._plain_projection = type(self).transform_qk is not PagedAttention.transform_qk

    def transform_qk(self, q: torch.Tensor, k: Optional[torch.Tensor], batch: Any) -> None:
        """The seam between projection and rotation: a subclass may change the projected queries
        `q` [T, Hq, hd] and keys `k` [T, Hkv, hd] (None when this call writes no cache) in place
        here (a norm per head, say) before they are rotated and the keys are cached.  Overriding it
        takes the step off the fused projection + rotation + cache-write kernel, and off captured
        steps unless the subclass sets `transform_replayable`.

        The elements of a head arrive in the order the kernels rotate them, which for a position
        encoding with the "halves" pairing is not the folder's: element j here is element
        `self.qk_order[j]` of the head as wq and wk give it (`qk_order` is the identity for adjacent
        pairs; it is set by `bind`).  A subclass with a tensor per element of a head (the weight of a
        norm) reorders it once, `weight[self.qk_order]`, after calling `bind` of this class."""

    transform_replayable = False  # whether an overriding `transform_qk` keeps to the rule of `Part.replayable`

    @property
    def replayable(self) -> bool:
        own = type(self).transform_qk is PagedAttention.transform_qk or self.transform_replayable
        return own and (self.position_encoding is None or self.position_encoding.replayable)

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        hd = self.head_dim
        q_out = self.n_heads * hd
        kv_out = self.n_kv_heads * hd
        table = self.position_encoding.rotary_table() if self.position_encoding is not None else None
        if write_cache and not self._plain_projection:
            qkv = ops.qkv_rope_write(
                x, self.qkv.weight, self.qkv.bias, self.n_heads, self.n_kv_heads, hd,
                batch.positions, table, cache.cache, cache.block_table, batch.seq_of_token, streamed=self.qkv.streamed,
            )
            q = qkv[:, :q_out].unflatten(1, (self.n_heads, hd))
        else:
            qkv = self.qkv(x)
            q = qkv[:, :q_out].unflatten(1, (self.n_heads, hd))
            if write_cache:
                k = qkv[:, q_out : q_out + kv_out].unflatten(1, (self.n_kv_heads, hd))
                v = qkv[:, q_out + kv_out :].unflatten(1, (self.n_kv_heads, hd))
                self.transform_qk(q, k, batch)
                ops.rope_kv_write(q, k, v, batch.positions, table, cache.cache, cache.block_table, batch.seq_of_token)
            else:
                # reads a cache that another layer wrote in this step: only the queries are needed
                self.transform_qk(q, None, batch)
                if table is not None:
                    ops.rope_kv_write(q, None, None, batch.positions, table)
        attn = ops.paged_attention(q, cache.cache, cache.block_table, batch, self.window, self.scale)
        return self.wo(attn, partials_ok=True)  # added into the residual by the next norm


register_part("mixer", "paged_attention", PagedAttention)


class SinkAttention(Mixer):
    """Grouped-query attention over a paged cache with a norm over the whole query and key projections, a softmax
    that holds a learned sink per head, and heads whose values may have another size than their queries and keys.

        q = W_q x, k = W_k x, v = W_v x                          no biases; `n_heads` heads of `qk_dim`, `n_kv_heads` of
                                                                 `qk_dim` (keys) and `v_dim` (values)
        q <- q / sqrt(mean(q^2) + eps) * w_q                     over all heads of the projection at once, before the
        k <- k / sqrt(mean(k^2) + eps) * w_k                     rotation (`qk_norm`; float32)
        rotation of q and k by the position encoding             its table may rotate fewer than qk_dim dimensions
        p_j = exp(scale * q . k_j) / (sum_i exp(scale * q . k_i) + exp(sink_h))   over the `window` keys up to the query's own
        out = W_o [sum_j p_j v_j of every head]

    The sink has no key and no value, is not scaled and counts once.  Keys and values are cached with one head size,
    the larger of qk_dim and v_dim rounded up to a multiple of 16 (zeros beyond a head's own size, which add nothing to a
    score and give output columns that W_o, widened by zero columns at load, ignores), so the attention kernels
    of equal key and value heads serve it.  `names` gives the tensors' local names for the roles q, k, v, o, q_norm,
    k_norm and sink."""

    replayable = True
    DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "sink": "sink"}

    def __init__(
        self,
        dim: int,
        n_heads: int,
        n_kv_heads: int,
        qk_dim: int,
        v_dim: int,
        scale: float,
        window: Optional[int] = None,
        qk_norm: bool = True,
        eps: float = 1e-6,
        sink: bool = True,
        position_encoding: Optional[PartChoice] = None,
        names: Optional[Mapping[str, str]] = None,
    ) -> None:
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"{n_heads} query heads do not divide into {n_kv_heads} key/value heads")
        head_dim = -(-max(qk_dim, v_dim) // 16) * 16
        if min(qk_dim, v_dim) < 1 or head_dim > MAX_HEAD_DIM:
            raise ValueError(f"heads of {qk_dim} (queries, keys) and {v_dim} (values) are outside 1..{MAX_HEAD_DIM}, the sizes the attention kernels take")
        if window is not None and window < 1:
            raise ValueError("a window holds at least the query's own key")
        self.dim, self.n_heads, self.n_kv_heads = dim, n_heads, n_kv_heads
        self.qk_dim, self.v_dim, self.head_dim = qk_dim, v_dim, head_dim
        self.scale, self.window, self.qk_norm, self.eps, self.sink = float(scale), window, qk_norm, float(eps), sink
        self.names = {**self.DEFAULT_NAMES, **dict(names or {})}
        self.position_encoding: Optional[PositionEncoding] = (
            position_encoding.build("position_encoding") if position_encoding is not None else None
        )

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, window=self.window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n = self.names
        q_out, k_out, v_out = self.n_heads * self.qk_dim, self.n_kv_heads * self.qk_dim, self.n_kv_heads * self.v_dim
        specs = {
            n["q"]: TensorSpec((q_out, self.dim)),
            n["k"]: TensorSpec((k_out, self.dim)),
            n["v"]: TensorSpec((v_out, self.dim)),
            n["o"]: TensorSpec((self.dim, self.n_heads * self.v_dim)),
        }
        if self.qk_norm:
            specs[n["q_norm"]] = TensorSpec((q_out,), init="norm", precision="stored")
            specs[n["k_norm"]] = TensorSpec((k_out,), init="norm", precision="stored")
        if self.sink:
            specs[n["sink"]] = TensorSpec((self.n_heads,), init="zeros", precision="stored")
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        n = self.names
        device = tensors[n["q"]].device
        self.qkv = LinearWeights.joined([tensors[n["q"]], tensors[n["k"]], tensors[n["v"]]], [None, None, None], stream_copy=runtime.stream_copies)
        wo = tensors[n["o"]]
        if self.v_dim != self.head_dim:
            # the attention kernels return heads of the cached size: columns of zeros where a head's values end
            wide = torch.zeros((self.dim, self.n_heads, self.head_dim), dtype=wo.dtype, device=device)
            wide[:, :, : self.v_dim] = wo.reshape(self.dim, self.n_heads, self.v_dim)
            wo = wide.reshape(self.dim, self.n_heads * self.head_dim)
        self.wo = LinearWeights(wo, stream_copy=runtime.stream_copies)
        self.q_weight = tensors[n["q_norm"]].float().contiguous() if self.qk_norm else None
        self.k_weight = tensors[n["k_norm"]].float().contiguous() if self.qk_norm else None
        self.sinks = tensors[n["sink"]].float().contiguous() if self.sink else None
        self.table: Optional[torch.Tensor] = None
        if self.position_encoding is not None:
            self.position_encoding.bind({}, runtime)
            if self.position_encoding.rotary_pairing() != "adjacent":
                raise ValueError("this mixer rotates adjacent pairs only")
            table = self.position_encoding.rotary_table()
            if table is not None:
                if 2 * table.numel() > self.qk_dim:
                    raise ValueError(f"{2 * table.numel()} rotated dimensions exceed the head's {self.qk_dim}")
                # a frequency of 0 leaves its pair alone: the head's other dimensions, and the padding
                self.table = torch.zeros(self.head_dim // 2, dtype=torch.float32, device=device)
                self.table[: table.numel()] = table.to(device)

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        qkv = self.qkv(x, partials_ok=True)
        q = ops.qk_norm_rope_write(
            qkv, self.n_heads, self.n_kv_heads, self.qk_dim, self.v_dim, self.head_dim, self.q_weight, self.k_weight, self.eps,
            batch.positions, self.table, self.runtime.act_dtype,
            cache.cache if write_cache else None, cache.block_table if write_cache else None, batch.seq_of_token if write_cache else None,
        )
        attn = ops.paged_attention(q, cache.cache, cache.block_table, batch, self.window, self.scale, sink=self.sinks)
        return self.wo(attn, partials_ok=True)  # added into the residual by the next norm


register_part("mixer", "sink_attention", SinkAttention)


class TalkingAttention(Mixer):
    """Grouped-query attention over a paged cache whose heads exchange their softmax weights, with biased projections,
    a sliding window and a sink in every head's softmax.

        q = W_q x + b_q, k = W_k x + b_k, v = W_v x + b_v        `n_heads` heads of `qk_dim`, `n_kv_heads` of `qk_dim` (keys)
                                                                 and `v_dim` (values); biases where `bias`
        rotation of q and k by the position encoding             its table may turn fewer than qk_dim dimensions, in
                                                                 adjacent pairs or in halves of the turned part
        p_g(j) = exp(scale q_g . k_j) / (sum_i exp(scale q_g . k_i) + exp(sink_g))    over the `window` keys up to the query's own
        w_h(j) = sum_g talk[h, g] p_g(j)                         where `talk`: the heads' weights mixed after the softmax
        out = W_o [sum_j w_h(j) v_j of every head, from h's own key/value head] + b_o

    The sink (where `sink`) is a learned score a head that enters the softmax's denominator only: nothing is read
    for it, the scale does not touch it, and the mixing of the heads leaves it out.  With
    `own_kv=False` the mixer has no key and value projections: it is run on a cache that another layer of equal
    key/value heads, sizes and rotation has written in the same step (`write_cache` false).  `cache_window` is what
    the cache keeps (default: `window`): a layer whose cache another layer reads through a longer window keeps that
    longer one.  Keys and values are cached with one head size, the larger of qk_dim and v_dim rounded up to a
    multiple of 16 (zeros beyond a head's own size; W_o is widened by zero columns at load).  Without `talk` the
    paged attention kernels of the other mixers serve it.  `names`: the tensors' local names for the roles q, k, v,
    o, q_bias, k_bias, v_bias, o_bias, sink and talk."""

    replayable = True
    DEFAULT_NAMES = {
        "q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "o_bias": "o.b",
        "sink": "sink", "talk": "talk",
    }
    _KEEP_WINDOW = object()

    def __init__(
        self,
        dim: int,
        n_heads: int,
        n_kv_heads: int,
        qk_dim: int,
        v_dim: int,
        scale: float,
        window: Optional[int] = None,
        cache_window: Any = _KEEP_WINDOW,
        bias: bool = True,
        sink: bool = True,
        talk: bool = True,
        own_kv: bool = True,
        position_encoding: Optional[PartChoice] = None,
        names: Optional[Mapping[str, str]] = None,
    ) -> None:
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"{n_heads} query heads do not divide into {n_kv_heads} key/value heads")
        head_dim = -(-max(qk_dim, v_dim) // 16) * 16
        if min(qk_dim, v_dim) < 1 or head_dim > MAX_HEAD_DIM:
            raise ValueError(f"heads of {qk_dim} (queries, keys) and {v_dim} (values) are outside 1..{MAX_HEAD_DIM}, the sizes the attention kernels take")
        if window is not None and window < 1:
            raise ValueError("a window holds at least the query's own key")
        if talk and n_heads > ops.MAX_TALK_HEADS:
            raise ValueError(f"{n_heads} heads that mix their weights: the kernel takes up to {ops.MAX_TALK_HEADS}")
        self.dim, self.n_heads, self.n_kv_heads = dim, n_heads, n_kv_heads
        self.qk_dim, self.v_dim, self.head_dim = qk_dim, v_dim, head_dim
        self.scale, self.window = float(scale), window
        self.cache_window = window if cache_window is self._KEEP_WINDOW else cache_window
        if self.cache_window is not None and (window is None or self.cache_window < window):
            raise ValueError("the cache must keep at least the keys of the mixer's own window")
        self.bias, self.sink, self.talk, self.own_kv = bias, sink, talk, own_kv
        self.names = {**self.DEFAULT_NAMES, **dict(names or {})}
        self.position_encoding: Optional[PositionEncoding] = (
            position_encoding.build("position_encoding") if position_encoding is not None else None
        )

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, window=self.cache_window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n = self.names
        q_out, k_out, v_out = self.n_heads * self.qk_dim, self.n_kv_heads * self.qk_dim, self.n_kv_heads * self.v_dim
        specs = {n["q"]: TensorSpec((q_out, self.dim)), n["o"]: TensorSpec((self.dim, self.n_heads * self.v_dim))}
        if self.own_kv:
            specs[n["k"]] = TensorSpec((k_out, self.dim))
            specs[n["v"]] = TensorSpec((v_out, self.dim))
        if self.bias:
            specs[n["q_bias"]] = TensorSpec((q_out,), precision="stored")
            specs[n["o_bias"]] = TensorSpec((self.dim,), precision="stored")
            if self.own_kv:
                specs[n["k_bias"]] = TensorSpec((k_out,), precision="stored")
                specs[n["v_bias"]] = TensorSpec((v_out,), precision="stored")
        if self.sink:
            specs[n["sink"]] = TensorSpec((self.n_heads,), init="zeros", precision="stored")
        if self.talk:
            specs[n["talk"]] = TensorSpec((self.n_heads, self.n_heads), init="identity", precision="stored")
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        n = self.names
        roles = ("q", "k", "v") if self.own_kv else ("q",)
        weights = {r: tensors[n[r]] for r in roles}
        biases = {r: (tensors[n[r + "_bias"]].float() if self.bias else None) for r in roles}
        device = weights["q"].device
        self.table: Optional[torch.Tensor] = None
        if self.position_encoding is not None:
            self.position_encoding.bind({}, runtime)
            table = self.position_encoding.rotary_table()
            if table is not None:
                turned = 2 * table.numel()
                if turned > self.qk_dim:
                    raise ValueError(f"{turned} rotated dimensions exceed the head's {self.qk_dim}")
                if self.position_encoding.rotary_pairing() == "halves":
                    # the kernels turn adjacent elements: bring element i and i + turned / 2 of every query and key head
                    # side by side, once, by the order of the projections' rows (a layer that reads another's cache
                    # turns with the same table, so its queries meet that layer's keys in the same order)
                    half = turned // 2
                    order = torch.cat([torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1), torch.arange(turned, self.qk_dim)]).to(device)
                    for r, heads in (("q", self.n_heads), ("k", self.n_kv_heads)):
                        if r not in weights:
                            continue
                        rows = (torch.arange(heads, device=device)[:, None] * self.qk_dim + order[None, :]).reshape(-1)
                        weights[r] = weights[r][rows]
                        if biases[r] is not None:
                            biases[r] = biases[r][rows]
                # a frequency of 0 leaves its pair alone: the head's other dimensions, and the padding
                self.table = torch.zeros(self.head_dim // 2, dtype=torch.float32, device=device)
                self.table[: table.numel()] = table.to(device)
        self.proj = LinearWeights.joined([weights[r] for r in roles], [biases[r] for r in roles], stream_copy=runtime.stream_copies)
        wo = tensors[n["o"]]
        if self.v_dim != self.head_dim:
            # the attention kernels return heads of the cached size: columns of zeros where a head's values end
            wide = torch.zeros((self.dim, self.n_heads, self.head_dim), dtype=wo.dtype, device=device)
            wide[:, :, : self.v_dim] = wo.reshape(self.dim, self.n_heads, self.v_dim)
            wo = wide.reshape(self.dim, self.n_heads * self.head_dim)
        self.wo = LinearWeights(wo, tensors[n["o_bias"]].float() if self.bias else None, stream_copy=runtime.stream_copies)
        self.sinks = tensors[n["sink"]].float().contiguous() if self.sink else None
        self.talk_matrix = tensors[n["talk"]].float().contiguous() if self.talk else None

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        if write_cache != self.own_kv:
            raise ValueError("a mixer with key and value projections writes its cache, one without reads another layer's")
        proj = self.proj(x)
        q = ops.qk_norm_rope_write(
            proj, self.n_heads, self.n_kv_heads if self.own_kv else 0, self.qk_dim, self.v_dim, self.head_dim, None, None, 1.0,
            batch.positions, self.table, self.runtime.act_dtype,
            cache.cache if write_cache else None, cache.block_table if write_cache else None, batch.seq_of_token if write_cache else None,
        )
        if self.talk_matrix is not None:
            attn = ops.talking_attention(q, cache.cache, cache.block_table, batch, self.window, self.scale, sink=self.sinks, talk=self.talk_matrix)
        else:
            attn = ops.paged_attention(q, cache.cache, cache.block_table, batch, self.window, self.scale, sink=self.sinks)
        return self.wo(attn, partials_ok=self.wo.bias is None)  # added into the residual by the next norm


register_part("mixer", "talking_attention", TalkingAttention)


class HeadNormAttention(Mixer):
    """Grouped-query attention over a paged cache with a norm of every query and key head, a cap on the scores, an
    output gate, and optionally values blended with those of an earlier layer.

        q = W_q x + b_q, k = W_k x + b_k, v = W_v x + b_v        `n_heads` heads of `qk_dim`, `n_kv_heads` of `qk_dim` (keys)
                                                                 and `v_dim` (values); biases where `bias`
        q_h <- q_h / sqrt(mean(q_h^2) + eps) * w_q, k likewise   per head, one weight of qk_dim values for all heads
                                                                 (`qk_norm`; float32), before the rotation
        rotation of q and k by the position encoding             its table may turn fewer than qk_dim dimensions, in
                                                                 adjacent pairs or in halves of the turned part
        v <- (1 - lam) v + lam v_source                          `value_mix="mix"`: v_source are the values that the layer
                                                                 with `value_mix="source"` and the same `value_mix_key`
                                                                 made of the same tokens in this step; lam is a stored
                                                                 scalar; the blended v is what is cached
        s_j = scale q . k_j;  s_j <- softcap tanh(s_j / softcap) where `softcap`
        softmax over the keys j <= i that the mask leaves: the last `window` keys (own included), or, with `chunk`, the keys
            of the query's own block of `chunk` positions counted from the start of the sequence; neither: all
        out = W_o ([sum_j p_j v_j of every head] * sigmoid(W_g x))   the gate where `gate`, element by element

    Keys and values are cached with one head size, the larger of qk_dim and v_dim rounded up to a multiple of 16 (zeros
    beyond a head's own size; W_o and W_g are widened by zero columns and rows at load), so the attention kernels of
    equal key and value heads serve it.  `names` gives the tensors' local names for the roles q, k, v, o, g, q_bias,
    k_bias, v_bias, q_norm, k_norm and value_mix."""

    replayable = True
    DEFAULT_NAMES = {
        "q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
        "q_norm": "q.norm", "k_norm": "k.norm", "value_mix": "vmix",
    }

    def __init__(
        self,
        dim: int,
        n_heads: int,
        n_kv_heads: int,
        qk_dim: int,
        v_dim: int,
        scale: float,
        window: Optional[int] = None,
        chunk: Optional[int] = None,
        softcap: Optional[float] = None,
        bias: bool = True,
        qk_norm: bool = True,
        eps: float = 1e-6,
        gate: bool = True,
        value_mix: Optional[str] = None,
        value_mix_key: str = "values",
        position_encoding: Optional[PartChoice] = None,
        names: Optional[Mapping[str, str]] = None,
    ) -> None:
        if n_heads % n_kv_heads != 0:
            raise ValueError(f"{n_heads} query heads do not divide into {n_kv_heads} key/value heads")
        head_dim = -(-max(qk_dim, v_dim) // 16) * 16
        if min(qk_dim, v_dim) < 1 or head_dim > MAX_HEAD_DIM:
            raise ValueError(f"heads of {qk_dim} (queries, keys) and {v_dim} (values) are outside 1..{MAX_HEAD_DIM}, the sizes the attention kernels take")
        if window is not None and chunk is not None:
            raise ValueError("a window and blocks of positions exclude each other")
        if (window is not None and window < 1) or (chunk is not None and chunk < 1):
            raise ValueError("a window or a block holds at least the query's own key")
        if softcap is not None and not softcap > 0:
            raise ValueError("a cap on the scores must be positive")
        if value_mix not in (None, "source", "mix"):
            raise ValueError(f"value_mix {value_mix!r}: None, 'source' and 'mix' are known")
        self.dim, self.n_heads, self.n_kv_heads = dim, n_heads, n_kv_heads
        self.qk_dim, self.v_dim, self.head_dim = qk_dim, v_dim, head_dim
        self.scale, self.window, self.chunk, self.softcap = float(scale), window, chunk, (float(softcap) if softcap is not None else None)
        self.bias, self.qk_norm, self.eps, self.gate = bias, qk_norm, float(eps), gate
        self.value_mix, self.value_mix_key = value_mix, value_mix_key
        self.names = {**self.DEFAULT_NAMES, **dict(names or {})}
        self.position_encoding: Optional[PositionEncoding] = (
            position_encoding.build("position_encoding") if position_encoding is not None else None
        )

    def cache_spec(self) -> PagedKVSpec:
        if self.chunk is not None:
            return ChunkedKVSpec(n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, chunk=self.chunk)
        return PagedKVSpec(n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, window=self.window)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        n = self.names
        q_out, k_out, v_out = self.n_heads * self.qk_dim, self.n_kv_heads * self.qk_dim, self.n_kv_heads * self.v_dim
        specs = {
            n["q"]: TensorSpec((q_out, self.dim)),
            n["k"]: TensorSpec((k_out, self.dim)),
            n["v"]: TensorSpec((v_out, self.dim)),
            n["o"]: TensorSpec((self.dim, self.n_heads * self.v_dim)),
        }
        if self.bias:
            specs[n["q_bias"]] = TensorSpec((q_out,), precision="stored")
            specs[n["k_bias"]] = TensorSpec((k_out,), precision="stored")
            specs[n["v_bias"]] = TensorSpec((v_out,), precision="stored")
        if self.qk_norm:
            specs[n["q_norm"]] = TensorSpec((self.qk_dim,), init="norm", precision="stored")
            specs[n["k_norm"]] = TensorSpec((self.qk_dim,), init="norm", precision="stored")
        if self.gate:
            specs[n["g"]] = TensorSpec((self.n_heads * self.v_dim, self.dim))
        if self.value_mix is not None:  # the source layer stores the scalar too and does not use it
            specs[n["value_mix"]] = TensorSpec((), init="zeros", precision="stored")
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        n = self.names
        wq, wk, wv, wo = tensors[n["q"]], tensors[n["k"]], tensors[n["v"]], tensors[n["o"]]
        device = wq.device
        biases = [tensors[n[r]].float() for r in ("q_bias", "k_bias", "v_bias")] if self.bias else None
        q_weight = tensors[n["q_norm"]].float() if self.qk_norm else None
        k_weight = tensors[n["k_norm"]].float() if self.qk_norm else None
        self.table: Optional[torch.Tensor] = None
        if self.position_encoding is not None:
            self.position_encoding.bind({}, runtime)
            table = self.position_encoding.rotary_table()
            if table is not None:
                turned = 2 * table.numel()
                if turned > self.qk_dim:
                    raise ValueError(f"{turned} rotated dimensions exceed the head's {self.qk_dim}")
                if self.position_encoding.rotary_pairing() == "halves":
                    # the kernels turn adjacent elements: bring element i and i + turned / 2 of every query and key head
                    # side by side, once, by the order of the projections' rows (and of what else is stored per element)
                    half = turned // 2
                    order = torch.cat([torch.stack([torch.arange(half), torch.arange(half) + half], dim=1).reshape(-1), torch.arange(turned, self.qk_dim)]).to(device)
                    rows_q = (torch.arange(self.n_heads, device=device)[:, None] * self.qk_dim + order[None, :]).reshape(-1)
                    rows_k = (torch.arange(self.n_kv_heads, device=device)[:, None] * self.qk_dim + order[None, :]).reshape(-1)
                    wq, wk = wq[rows_q], wk[rows_k]
                    if biases is not None:
                        biases[0], biases[1] = biases[0][rows_q], biases[1][rows_k]
                    if self.qk_norm:
                        q_weight, k_weight = q_weight[order], k_weight[order]
                # a frequency of 0 leaves its pair alone: the head's other dimensions, and the padding
                self.table = torch.zeros(self.head_dim // 2, dtype=torch.float32, device=device)
                self.table[: table.numel()] = table.to(device)
        matrices = [wq, wk, wv]
        if self.gate:
            wg = tensors[n["g"]]
            if self.v_dim != self.head_dim:  # the gate meets heads of the cached size
                wide = torch.zeros((self.n_heads, self.head_dim, self.dim), dtype=wg.dtype, device=device)
                wide[:, : self.v_dim] = wg.reshape(self.n_heads, self.v_dim, self.dim)
                wg = wide.reshape(self.n_heads * self.head_dim, self.dim)
            matrices.append(wg)
        self.proj = LinearWeights.joined(matrices, [None] * len(matrices), stream_copy=runtime.stream_copies)
        self.qkv_width = wq.shape[0] + wk.shape[0] + wv.shape[0]
        self.qkv_bias = torch.cat(biases).contiguous() if biases is not None else None
        self.q_weight = q_weight.contiguous() if q_weight is not None else None
        self.k_weight = k_weight.contiguous() if k_weight is not None else None
        if self.v_dim != self.head_dim:
            wide = torch.zeros((self.dim, self.n_heads, self.head_dim), dtype=wo.dtype, device=device)
            wide[:, :, : self.v_dim] = wo.reshape(self.dim, self.n_heads, self.v_dim)
            wo = wide.reshape(self.dim, self.n_heads * self.head_dim)
        self.wo = LinearWeights(wo, stream_copy=runtime.stream_copies)
        self.lam = tensors[n["value_mix"]].float().reshape(1).contiguous() if self.value_mix == "mix" else None

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        if not write_cache:
            raise ValueError("this mixer writes its own cache")
        proj = self.proj(x, partials_ok=not self.gate)
        key = ("value_mix", self.value_mix_key)
        v_other = None
        if self.value_mix == "mix":
            v_other = batch.scratch.get(key)
            if v_other is None:
                raise RuntimeError(f"no layer has left the values {self.value_mix_key!r} in this step")
        result = ops.head_norm_rope_write(
            proj, self.n_heads, self.n_kv_heads, self.qk_dim, self.v_dim, self.head_dim, self.qkv_bias, self.q_weight, self.k_weight,
            self.eps, batch.positions, self.table, self.runtime.act_dtype, cache.cache, cache.block_table, batch.seq_of_token,
            v_other=v_other, v_mix=self.lam, keep_values=self.value_mix == "source",
        )
        if self.value_mix == "source":
            q, batch.scratch[key] = result
        else:
            q = result
        attn = ops.paged_attention(q, cache.cache, cache.block_table, batch, self.window, self.scale, softcap=self.softcap, chunk=self.chunk)
        if self.gate:
            attn = ops.sigmoid_mul(attn, proj[:, self.qkv_width :])
        return self.wo(attn, partials_ok=True)  # added into the residual by the next norm


register_part("mixer", "head_norm_attention", HeadNormAttention)


class SideBySide(Mixer):
    """Several mixers that read the same input; the result is the sum of theirs, each times a constant:
    sum_i scale_i mixer_i(x).  `mixers` maps a name to (the mixer chosen, its factor); a child's tensors carry its
    name and a dot before their own.  Every child keeps a cache or state of its own (`children()` lists them in the
    order in which `forward` takes their views); the sum is left to whoever adds the result into the residual (an
    `ops.ScaledSum`)."""

    def __init__(self, mixers: Mapping[str, Any]) -> None:
        if not mixers:
            raise ValueError("at least one mixer is needed")
        self.names = list(mixers)
        self.parts = [mixers[name][0].build("mixer") for name in self.names]
        self.scales = [float(mixers[name][1]) for name in self.names]

    @property
    def replayable(self) -> bool:
        return all(part.replayable for part in self.parts)

    def children(self):
        return list(self.parts)

    def cache_spec(self):
        raise TypeError("mixers side by side have a cache each; the block asks `children()`")

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {f"{name}.{t}": spec for name, part in zip(self.names, self.parts) for t, spec in part.tensor_specs().items()}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        for name, part in zip(self.names, self.parts):
            prefix = name + "."
            part.bind({t[len(prefix):]: v for t, v in tensors.items() if t.startswith(prefix)}, runtime)

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> Any:
        views = cache if isinstance(cache, tuple) else (cache,)
        if len(views) != len(self.parts):
            raise ValueError(f"{len(self.parts)} mixers side by side were given {len(views)} caches")
        return ops.ScaledSum([(part.forward(x, batch, view, write_cache), scale) for part, view, scale in zip(self.parts, views, self.scales)])


register_part("mixer", "side_by_side", SideBySide)
