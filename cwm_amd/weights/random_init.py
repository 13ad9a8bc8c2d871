"""Random weights from a configuration and a seed, and the writer of a model
folder (config.json + model.safetensors) that holds them.

The reference has no initialisation for generation: without a checkpoint its
parameters are uninitialised memory (cwm/fastgen/utils/loading.py:30,44-55).  Here
every tensor is drawn from a generator seeded by (seed, tensor name), so any subset
of a model can be reproduced alone: matrices and the embedding N(0, std), norm
weights 1 or U(0.5, 1.5), biases N(0, std).
"""

from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict, Mapping, Optional

import torch

from ..config.registry import parse_config
from ..config.schema import to_dict
from ..parts.base import TensorSpec


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(
    name: str,
    spec: TensorSpec,
    seed: int,
    std: float,
    norm_init: str,
    dtype: torch.dtype,
    device: torch.device = torch.device("cpu"),
) -> torch.Tensor:
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    shape = spec.drawn_shape()
    if spec.kind == "int":
        return torch.zeros(shape, dtype=torch.int32, device=device)
    if spec.init == "norm":
        if norm_init == "ones":
            t = torch.ones(shape, dtype=torch.float32, device=device)
        elif norm_init == "uniform":
            t = torch.rand(shape, generator=gen, dtype=torch.float32, device=device) + 0.5
        else:
            raise ValueError(f"norm_init must be 'ones' or 'uniform', found {norm_init!r}")
    elif spec.init == "zeros":
        t = torch.zeros(shape, dtype=torch.float32, device=device)
    elif spec.init == "ones":
        t = torch.ones(shape, dtype=torch.float32, device=device)
    elif spec.init == "identity":
        t = torch.eye(shape[0], shape[1], dtype=torch.float32, device=device)
    else:
        t = torch.randn(shape, generator=gen, dtype=torch.float32, device=device) * std
    return t.to(dtype)


def random_tensors(
    specs: Mapping[str, TensorSpec],
    seed: int,
    std: float = 0.02,
    norm_init: str = "ones",
    dtype: torch.dtype = torch.bfloat16,
    device: torch.device = torch.device("cpu"),
) -> Dict[str, torch.Tensor]:
    return {name: random_tensor(name, spec, seed, std, norm_init, dtype, device) for name, spec in specs.items()}


def write_random_model(
    folder: str,
    config: Mapping[str, Any],
    seed: int,
    std: float = 0.02,
    norm_init: str = "ones",
    dtype: Optional[str] = None,
) -> None:
    """Write `folder/config.json` and `folder/model.safetensors` for `config` (a
    config.json dictionary with its `architecture` key).  `dtype` ("bfloat16" or
    "float32") is the stored type; it defaults to the configuration's own."""
    from safetensors.torch import save_file

    from ..models.model import Model

    arch, typed = parse_config(config)
    if dtype is None:
        dtype = getattr(typed, "dtype", "bfloat16")
    torch_dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype]
    model = Model(arch.build_plan(typed))
    tensors = random_tensors(model.tensor_specs(), seed, std=std, norm_init=norm_init, dtype=torch_dtype)
    os.makedirs(folder, exist_ok=True)
    full = to_dict(typed)
    if "dtype" in full:
        full["dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(full, fh, indent=2)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
