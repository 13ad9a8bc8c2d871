"""The Digasun decoder as a plan of parts.

Layers whose two sublayers read one layer norm (weight and bias) of the residual, each through a short causal
convolution of its own, and join the residual in one sum; after it every layer adds its own gated input from the
token's side embedding.  The mixer is an attention (biased projections, partial rotation in halves, a sliding window,
a sink in the softmax, the heads' weights mixed after the softmax; a layer may read an earlier layer's keys and
values instead of making its own) or a gated linear attention; the feed-forward is dense and gated with a clamped
activation, or routed experts with a biased router and a gated shared expert.  The final norm is a layer norm.
Tensor names: `embed`, `side.embed`, `l<i>.norm1`, `l<i>.norm1.b`, `l<i>.canon1`, `l<i>.canon2`,
`l<i>.mix.{q,q.b,k,k.b,v,v.b,o,o.b,sink,talk}` or `l<i>.mix.{q,k,v,g,o,norm,a1,a2,a2.b}`,
`l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{router,router.b,e<j>.{gate,up,down},shared.{gate,up,down,sg}}`,
`l<i>.side.{gate,proj,norm}`, `final.norm`, `final.norm.b`, `head`.
"""

from __future__ import annotations

from typing import Dict, Optional

from ..config.digasun import AttentionConfig, DigasunConfig, FeedForwardConfig, LinearAttentionConfig
from ..config.registry import register_architecture
from ..parts.base import LayerCall, LayerPlan, ModelPlan, PartChoice, PartSlot

ARCHITECTURE_NAME = "Digasun"
DENSE_ALPHA = 1.702  # the slope inside the dense feed-forward's sigmoid: the design fixes it


def _attention(width: int, sizes: AttentionConfig, cache_window: Optional[int]) -> PartChoice:
    rotation = None
    if sizes.rot is not None and sizes.rot.dims > 0:
        rotation = PartChoice("rotary", {"head_dim": sizes.rot.dims, "theta": sizes.rot.base, "pairing": "halves"})
    return PartChoice(
        "talking_attention",
        {
            "dim": width, "n_heads": sizes.heads, "n_kv_heads": sizes.kv_heads, "qk_dim": sizes.dim, "v_dim": sizes.vdim,
            "scale": sizes.scale, "window": sizes.mask.size if sizes.mask is not None else None, "cache_window": cache_window,
            "bias": True, "sink": True, "talk": True, "own_kv": sizes.kv_from is None, "position_encoding": rotation,
        },
    )


def _feed_forward(width: int, mlp: FeedForwardConfig) -> PartChoice:
    if mlp.kind == "dense":
        return PartChoice(
            "gated_mlp", {"dim": width, "hidden_dim": mlp.ff, "activation": "clamped_swish", "act_alpha": DENSE_ALPHA, "act_limit": mlp.limit},
        )
    shared = None
    if mlp.shared is not None:
        shared = PartChoice("gated_mlp", {"dim": width, "hidden_dim": mlp.shared.ff, "activation": "silu", "row_gate": "sg"})
    return PartChoice(
        "routed_experts",
        {
            "dim": width, "hidden_dim": mlp.expert.ff, "n_experts": mlp.router.experts, "top": mlp.router.top,
            "router_bias": True, "shared": shared, "shared_prefix": "shared.",
        },
    )


def cache_windows(config: DigasunConfig) -> Dict[int, Optional[int]]:
    """For every attention layer with keys and values of its own: the longest window through which it or a layer that
    reads its cache looks back (None: all keys), which is what its cache keeps."""
    spans: Dict[int, Optional[int]] = {}
    for i, layer in enumerate(config.layers):
        m = layer.mixer_config()
        if not isinstance(m, AttentionConfig):
            continue
        owner = i if m.kv_from is None else m.kv_from
        size = m.mask.size if m.mask is not None else None
        if owner not in spans:
            spans[owner] = size
        elif spans[owner] is not None:
            spans[owner] = None if size is None else max(spans[owner], size)
    return spans


def build_plan(config: DigasunConfig) -> ModelPlan:
    width, eps = config.width, config.norm.eps
    norm = PartChoice("layernorm", {"dim": width, "eps": eps, "tensor": "", "bias_tensor": ".b"})
    spans = cache_windows(config)
    layers, order = [], []
    for i, layer in enumerate(config.layers):
        sizes = layer.mixer_config()
        call = LayerCall(layer=i)
        parts = {"norm": PartSlot("norm", norm, "norm1")}
        if config.canon is not None:
            names = ("canon1", "canon2") if layer.mlp is not None else ("canon1",)
            ignored = () if layer.mlp is not None else ("canon2",)
            parts["conv"] = PartSlot("mixer", PartChoice("input_convolution", {"dim": width, "taps": config.canon.taps, "outputs": names, "ignored": ignored}), "")
        if isinstance(sizes, AttentionConfig):
            owner = i if sizes.kv_from is None else sizes.kv_from
            mixer = _attention(width, sizes, spans[owner])
            if sizes.kv_from is not None:
                # the attention reads the other layer's cache; the convolution before it keeps a state of its own
                call = LayerCall(layer=i, cache_of=sizes.kv_from, shared_mixers=(1 if config.canon is not None else 0,))
        elif isinstance(sizes, LinearAttentionConfig):
            mixer = PartChoice(
                "gated_linear_attention",
                {"dim": width, "heads": sizes.heads, "head_dim": sizes.dim, "v_dim": sizes.vdim, "tau": sizes.tau, "decay_rank": None, "eps": eps},
            )
        else:  # pragma: no cover  (LayerConfig has refused it)
            raise TypeError(f"layer {i}: no part for {type(sizes).__name__}")
        parts["mixer"] = PartSlot("mixer", mixer, "mix.")
        if layer.mlp is not None:
            parts["feed_forward"] = PartSlot("feed_forward", _feed_forward(width, layer.mlp), "mlp.")
        if config.token_side is not None:
            parts["token_input"] = PartSlot(
                "token_input",
                PartChoice(
                    "gated_token_side",
                    {"vocab_size": config.vocab, "dim": width, "side_dim": config.token_side.dim, "index": i, "n_parts": len(config.layers), "eps": eps},
                ),
                "side.",
            )
        layers.append(LayerPlan(prefix=f"l{i}.", block="shared_norm_parallel", parts=parts))
        order.append(call)
    sizes = {"vocab_size": config.vocab, "dim": width, "tensor": ""}
    scale = config.embedding.scale if config.embedding is not None else None
    return ModelPlan(
        vocab_size=config.vocab,
        dim=width,
        layers=layers,
        run_order=order,
        embedding=PartSlot("embedding", PartChoice("token_embedding", {**sizes, "scale": scale}), "embed"),
        final_norm=PartSlot("norm", norm, "final.norm"),
        head=PartSlot("head", PartChoice("linear_head", sizes), "head"),
        max_positions=config.max_positions,
    )


register_architecture(ARCHITECTURE_NAME, DigasunConfig, build_plan)
