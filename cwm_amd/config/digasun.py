"""Typed configuration of the Digasun decoder.

config.json names the vocabulary, the width, one eps for every norm, the embedding's scale, the taps of the input
convolutions (`canon`), the size of the per-layer token input (`token_side`) and a list of layers.  Every layer names
its mixer (`type`: "attention" or "gla"), the mixer's sizes (`mixer`) and its feed-forward (`mlp`, null for none;
`kind` "dense" or "moe").  Strict as every configuration: an unknown key is an error that names it.
"""

from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Any, List, Mapping, Optional

from .schema import ConfigError, from_dict


@dataclass(frozen=True)
class NormConfig:
    eps: float

    def __post_init__(self) -> None:
        if self.eps <= 0:
            raise ConfigError("norm.eps must be positive")


@dataclass(frozen=True)
class EmbeddingConfig:
    scale: float = 1.0


@dataclass(frozen=True)
class CanonConfig:
    taps: int  # inputs a convolution reads, the current one included

    def __post_init__(self) -> None:
        if self.taps < 1:
            raise ConfigError("canon.taps must be at least 1")


@dataclass(frozen=True)
class TokenSideConfig:
    dim: int  # elements of a token's side embedding that one layer reads

    def __post_init__(self) -> None:
        if self.dim < 1:
            raise ConfigError("token_side.dim must be positive")


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int

    def __post_init__(self) -> None:
        if self.dims < 0 or self.dims % 2 != 0:
            raise ConfigError("rot.dims must be even and not negative")
        if self.base <= 0:
            raise ConfigError("rot.base must be positive")


@dataclass(frozen=True)
class MaskConfig:
    size: int  # keys a query reads, its own included

    def __post_init__(self) -> None:
        if self.size < 1:
            raise ConfigError("mask.size must be at least 1")


@dataclass(frozen=True)
class AttentionConfig:
    """`heads` query heads on `kv_heads` key/value heads; queries and keys of `dim`, values of `vdim` per head.
    `kv_from`: the layer whose cached keys and values this layer reads instead of making its own."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotationConfig] = None
    mask: Optional[MaskConfig] = None
    kv_from: Optional[int] = None

    def __post_init__(self) -> None:
        if min(self.heads, self.kv_heads, self.dim, self.vdim) < 1:
            raise ConfigError("an attention mixer's sizes must be positive")
        if self.heads % self.kv_heads != 0:
            raise ConfigError(f"{self.heads} query heads do not divide into {self.kv_heads} key/value heads")
        if self.rot is not None and self.rot.dims > self.dim:
            raise ConfigError(f"rot.dims {self.rot.dims} exceeds the head's {self.dim} dimensions")
        if self.scale <= 0:
            raise ConfigError("scale must be positive")


@dataclass(frozen=True)
class LinearAttentionConfig:
    """Gated linear attention: `heads` heads with a state of `dim` x `vdim` each; a decay is sigmoid(.)^(1 / tau)."""

    heads: int
    dim: int
    vdim: int
    tau: float

    def __post_init__(self) -> None:
        if min(self.heads, self.dim, self.vdim) < 1 or not self.tau > 0:
            raise ConfigError("a gated linear attention needs positive sizes and a positive tau")


@dataclass(frozen=True)
class RouterConfig:
    experts: int
    top: int

    def __post_init__(self) -> None:
        if not 1 <= self.top <= self.experts:
            raise ConfigError(f"router: {self.top} experts a token out of {self.experts}")


@dataclass(frozen=True)
class ExpertConfig:
    ff: int

    def __post_init__(self) -> None:
        if self.ff < 1:
            raise ConfigError("an expert's ff must be positive")


@dataclass(frozen=True)
class FeedForwardConfig:
    """`kind` "dense": `ff` and `limit`.  `kind` "moe": `router`, `expert` and optionally `shared`."""

    kind: str
    ff: Optional[int] = None
    limit: Optional[float] = None
    router: Optional[RouterConfig] = None
    expert: Optional[ExpertConfig] = None
    shared: Optional[ExpertConfig] = None

    def __post_init__(self) -> None:
        if self.kind == "dense":
            if self.ff is None or self.ff < 1 or self.limit is None or not self.limit > 0:
                raise ConfigError("a dense mlp needs a positive ff and a positive limit")
            if self.router is not None or self.expert is not None or self.shared is not None:
                raise ConfigError("a dense mlp has no router and no experts")
        elif self.kind == "moe":
            if self.router is None or self.expert is None:
                raise ConfigError("an mlp of kind 'moe' needs router and expert")
            if self.ff is not None or self.limit is not None:
                raise ConfigError("an mlp of kind 'moe' has its sizes under expert and shared")
        else:
            raise ConfigError(f"mlp.kind {self.kind!r}: 'dense' and 'moe' are known")


MIXER_CONFIGS = {"attention": AttentionConfig, "gla": LinearAttentionConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any
    mlp: Optional[FeedForwardConfig] = None

    def __post_init__(self) -> None:
        self.mixer_config()  # reject what does not fit now, by key

    def kind(self) -> str:
        return re.sub(r"_\d+$", "", self.type)  # a numeric suffix marks another set of sizes of the same mixer

    def mixer_config(self):
        kind = self.kind()
        if kind not in MIXER_CONFIGS:
            raise ConfigError(f"layer type {self.type!r}: known mixers are {', '.join(sorted(MIXER_CONFIGS))}")
        if not isinstance(self.mixer, Mapping):
            raise ConfigError(f"the sizes of mixer {self.type!r} must be an object")
        return from_dict(MIXER_CONFIGS[kind], self.mixer, path="mixer")


@dataclass(frozen=True)
class DigasunConfig:
    architecture: str
    vocab: int
    width: int
    norm: NormConfig
    layers: List[LayerConfig]
    embedding: Optional[EmbeddingConfig] = None
    canon: Optional[CanonConfig] = None
    token_side: Optional[TokenSideConfig] = None
    max_positions: Optional[int] = None  # not a key of the design: only cache sizing reads it when given

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1:
            raise ConfigError("vocab and width must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        for i, layer in enumerate(self.layers):
            m = layer.mixer_config()
            if not isinstance(m, AttentionConfig) or m.kv_from is None:
                continue
            j = m.kv_from
            if not 0 <= j < i or self.layers[j].kind() != "attention":
                raise ConfigError(f"layer {i}: kv_from {j} must name an earlier attention layer")
            src = self.layers[j].mixer_config()
            if src.kv_from is not None:
                raise ConfigError(f"layer {i}: kv_from {j} names a layer without keys and values of its own")
            if (src.kv_heads, src.dim, src.vdim, src.rot) != (m.kv_heads, m.dim, m.vdim, m.rot):
                raise ConfigError(f"layer {i} reads layer {j}'s keys and values: their key/value heads, sizes and rotation must be equal")
