"""Typed configuration of the Dogotar decoder.

config.json names the vocabulary, the width, one eps for every norm and a list of layers.  Every layer names its
mixer (`type`: "attention", or "parallel" for an attention and a matrix memory side by side), the mixer's sizes
(`mixer`) and its feed-forward (`mlp`, null for none).  Strict as every configuration: an unknown key is an error
that names it.
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
class RotationScalingConfig:
    factor: float = 1.0  # every frequency is divided by it

    def __post_init__(self) -> None:
        if self.factor <= 0:
            raise ConfigError("rot.scaling.factor must be positive")


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int
    scaling: Optional[RotationScalingConfig] = None

    def __post_init__(self) -> None:
        if self.dims < 0 or self.dims % 2 != 0:
            raise ConfigError("rot.dims must be even and not negative")
        if self.base <= 0:
            raise ConfigError("rot.base must be positive")


@dataclass(frozen=True)
class MaskConfig:
    size: int  # an attention layer: keys a query reads, its own included; the attention beside a memory: positions of a block

    def __post_init__(self) -> None:
        if self.size < 1:
            raise ConfigError("mask.size must be at least 1")


@dataclass(frozen=True)
class AttentionConfig:
    """`heads` query heads and `kv_heads` key/value heads; queries and keys of `dim`, values of `vdim` per head."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float] = None
    rot: Optional[RotationConfig] = None
    mask: Optional[MaskConfig] = None
    v_mix: bool = False

    def __post_init__(self) -> None:
        if min(self.heads, self.kv_heads, self.dim, self.vdim) < 1:
            raise ConfigError("an attention mixer's sizes must be positive")
        if self.heads % self.kv_heads != 0:
            raise ConfigError(f"{self.heads} query heads do not divide into {self.kv_heads} key/value heads")
        if self.rot is not None and self.rot.dims > self.dim:
            raise ConfigError(f"rot.dims {self.rot.dims} exceeds the head's {self.dim} dimensions")
        if self.softcap is not None and self.softcap <= 0:
            raise ConfigError("softcap must be positive")
        if self.scale <= 0:
            raise ConfigError("scale must be positive")


@dataclass(frozen=True)
class MemoryConfig:
    """A matrix memory of `heads` heads, each `dim` x `vdim`, whose gates are capped at `gate_cap`."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float

    def __post_init__(self) -> None:
        if min(self.heads, self.dim, self.vdim) < 1 or self.gate_cap <= 0:
            raise ConfigError("a matrix memory needs positive sizes and a positive gate_cap")


@dataclass(frozen=True)
class ParallelConfig:
    """An attention (`left`) and a matrix memory (`right`) that read the same input; left_scale * left + right_scale * right."""

    left: AttentionConfig
    right: MemoryConfig
    left_scale: float = 1.0
    right_scale: float = 1.0


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str
    ff: int

    def __post_init__(self) -> None:
        if self.kind != "dense":
            raise ConfigError(f"mlp.kind {self.kind!r}: 'dense' is known")
        if self.ff < 1:
            raise ConfigError("mlp.ff must be positive")


MIXER_CONFIGS = {"attention": AttentionConfig, "parallel": ParallelConfig}


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
class DogotarConfig:
    architecture: str
    vocab: int
    width: int
    norm: NormConfig
    layers: List[LayerConfig]
    max_positions: Optional[int] = None  # not a key of the design: only cache sizing reads it when given

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1:
            raise ConfigError("vocab and width must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        sources = [layer.mixer_config() for layer in self.layers if layer.kind() == "attention"]
        sizes = {(m.kv_heads, m.vdim) for m in sources if m.v_mix}
        if len(sizes) > 1:
            raise ConfigError("layers that mix their values with the first such layer's need the same key/value heads and vdim")
