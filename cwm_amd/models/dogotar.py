"""The Dogotar decoder as a plan of parts.

Layers whose two sublayers read the same residual, each through a layer norm (weight and bias) of its own, and join it
in one sum.  The mixer is an attention (biased projections, a norm of every query and key head, partial rotation in
halves with linearly stretched positions, capped scores, a sliding window, values blended with those of the first
such layer, an output gate), or that attention's plainer form (no rotation, blocks of positions instead of a window,
no gate) side by side with a matrix memory; the feed-forward is dense with the tanh form of gelu.  The final norm is
a layer norm and the head is the embedding table.
Tensor names: `embed`, `l<i>.norm1`, `l<i>.norm1.b`, `l<i>.norm2`, `l<i>.norm2.b`,
`l<i>.mix.{q,q.b,k,k.b,v,v.b,q.norm,k.norm,vmix,g,o}` or `l<i>.mix.left.{q,q.b,k,k.b,v,v.b,q.norm,k.norm,o}` with
`l<i>.mix.right.{q,k,v,g,o,norm,i,i.b,f,f.b}`, `l<i>.mlp.{up,down}`, `final.norm`, `final.norm.b`.
"""

from __future__ import annotations

from ..config.dogotar import AttentionConfig, DogotarConfig, ParallelConfig
from ..config.registry import register_architecture
from ..parts.base import LayerCall, LayerPlan, ModelPlan, PartChoice, PartSlot

ARCHITECTURE_NAME = "Dogotar"


def _attention(width: int, eps: float, sizes: AttentionConfig, blocks: bool, gate: bool, value_mix) -> PartChoice:
    """`blocks`: mask.size is a block of positions rather than a window."""
    rotation = None
    if sizes.rot is not None and sizes.rot.dims > 0:
        factor = sizes.rot.scaling.factor if sizes.rot.scaling is not None else 1.0
        rotation = PartChoice("rotary", {"head_dim": sizes.rot.dims, "theta": sizes.rot.base, "linear_factor": factor, "pairing": "halves"})
    span = sizes.mask.size if sizes.mask is not None else None
    return PartChoice(
        "head_norm_attention",
        {
            "dim": width, "n_heads": sizes.heads, "n_kv_heads": sizes.kv_heads, "qk_dim": sizes.dim, "v_dim": sizes.vdim,
            "scale": sizes.scale, "window": None if blocks else span, "chunk": span if blocks else None, "softcap": sizes.softcap,
            "bias": True, "qk_norm": True, "eps": eps, "gate": gate, "value_mix": value_mix, "position_encoding": rotation,
        },
    )


def build_plan(config: DogotarConfig) -> ModelPlan:
    width, eps = config.width, config.norm.eps
    norm = PartChoice("layernorm", {"dim": width, "eps": eps, "tensor": "", "bias_tensor": ".b"})
    layers = []
    have_source = False
    for i, layer in enumerate(config.layers):
        sizes = layer.mixer_config()
        if isinstance(sizes, AttentionConfig):
            value_mix = None
            if sizes.v_mix:
                value_mix = "mix" if have_source else "source"
                have_source = True
            mixer = _attention(width, eps, sizes, blocks=False, gate=True, value_mix=value_mix)
        elif isinstance(sizes, ParallelConfig):
            left = _attention(width, eps, sizes.left, blocks=True, gate=False, value_mix=None)
            right = PartChoice(
                "matrix_memory",
                {"dim": width, "heads": sizes.right.heads, "head_dim": sizes.right.dim, "v_dim": sizes.right.vdim, "gate_cap": sizes.right.gate_cap, "eps": eps},
            )
            mixer = PartChoice("side_by_side", {"mixers": {"left": (left, sizes.left_scale), "right": (right, sizes.right_scale)}})
        else:  # pragma: no cover  (LayerConfig has refused it)
            raise TypeError(f"layer {i}: no part for {type(sizes).__name__}")
        parts = {"norm1": PartSlot("norm", norm, "norm1"), "mixer": PartSlot("mixer", mixer, "mix.")}
        if layer.mlp is not None:
            parts["norm2"] = PartSlot("norm", norm, "norm2")
            parts["feed_forward"] = PartSlot(
                "feed_forward", PartChoice("activated_mlp", {"dim": width, "hidden_dim": layer.mlp.ff, "activation": "gelu_tanh"}), "mlp.",
            )
        layers.append(LayerPlan(prefix=f"l{i}.", block="parallel_pre_norm", parts=parts))
    sizes = {"vocab_size": config.vocab, "dim": width, "tensor": ""}
    return ModelPlan(
        vocab_size=config.vocab,
        dim=width,
        layers=layers,
        run_order=[LayerCall(layer=i) for i in range(len(layers))],
        embedding=PartSlot("embedding", PartChoice("token_embedding", sizes), "embed"),
        final_norm=PartSlot("norm", norm, "final.norm"),
        head=PartSlot("head", PartChoice("linear_head", sizes), "embed"),
        max_positions=config.max_positions,
    )


register_architecture(ARCHITECTURE_NAME, DogotarConfig, build_plan)
