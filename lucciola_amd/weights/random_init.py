"""Random weights from a configuration and a seed.

The reference has no such mode (it only reads a checkpoint, src/qwen.cc:69-84).  Projections
and tables are N(0, std); norm weights are 1 + N(0, std) so that a norm applied in the wrong
place or left out changes the result.  Each tensor's generator is seeded from the seed and the
tensor's name, so values do not depend on the order in which tensors are made.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Any, Dict, Iterator, Mapping, Tuple

import torch

from .loader import ParamDecl
from .safetensors_io import write_safetensors


def _tensor_seed(seed: int, name: str) -> int:
    return (int(seed) * 0x9E3779B1 + zlib.crc32(name.encode("utf-8"))) & 0x7FFFFFFFFFFFFFFF


def random_tensors(declared: Mapping[str, ParamDecl], seed: int, std: float,
                   dtype: torch.dtype = torch.bfloat16,
                   device: str = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    """Yield ``(name, tensor)`` for every declared tensor; values are drawn in float32 and
    rounded to ``dtype`` once."""
    dev = torch.device(device)
    for name, decl in declared.items():
        if decl.role == "int":
            yield name, torch.zeros(decl.shape, dtype=torch.int32, device=dev)
            continue
        gen = torch.Generator(device=dev)
        gen.manual_seed(_tensor_seed(seed, name))
        if decl.init == "zeros":
            t = torch.zeros(decl.shape, dtype=torch.float32, device=dev)
        elif decl.init == "ones":
            t = torch.ones(decl.shape, dtype=torch.float32, device=dev)
        else:
            t = torch.randn(decl.shape, generator=gen, dtype=torch.float32, device=dev) * std
            if decl.init == "ones_plus_normal":
                t += 1.0
            elif decl.init != "normal":
                raise ValueError(f"tensor '{name}': unknown init '{decl.init}'")
        yield name, t.to(dtype)


def write_model_folder(folder: str, config_dict: Dict[str, Any], seed: int,
                       dtype: torch.dtype = torch.bfloat16, std: float = None) -> str:
    """Make ``folder`` a model folder: config.json and model.safetensors with random weights
    for the architecture that ``config_dict`` names."""
    from ..config.registry import architecture_for
    from ..models.causal_lm import declared_tensors

    arch = architecture_for(config_dict)
    config = arch.read_config(config_dict)
    spec = arch.model_spec(config)
    declared = declared_tensors(spec)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(config_dict, fh, indent=2)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      random_tensors(declared, seed, spec.init_std if std is None else std, dtype))
    return folder
