"""From a model folder (or a configuration and a seed) to a model on the GPU."""
from __future__ import annotations

from typing import Any, Dict, Optional

import torch

from .. import models  # noqa: F401  (registers the architectures)
from ..config.engine_config import parse_dtype
from ..config.model_config import read_config_json
from ..config.registry import architecture_for
from ..config.specs import ModelSpec
from ..models.causal_lm import CausalLM, declared_tensors
from ..weights.loader import DictSource, FolderSource, WeightSource
from ..weights.random_init import random_tensors
from dataclasses import replace


def _build(spec: ModelSpec, source: WeightSource, dtype, device) -> CausalLM:
    optional = ()
    names = set(source.names())
    if spec.head_name is not None and spec.head_name not in names:
        # no separate head in the checkpoint: the head uses the embedding table, as the
        # reference does when lm_head.weight is absent (src/qwen.cc:80-84)
        spec = replace(spec, head_name=None)
    elif spec.head_name is None:
        optional = ("lm_head.weight",)
    try:
        return CausalLM(spec, source, parse_dtype(dtype), device, optional_names=optional)
    finally:
        source.close()


def load_model(folder: str, dtype="bfloat16", device="cuda:0"):
    """The model that ``folder``'s config.json names, with the weights of its
    model.safetensors.  Returns (model, typed configuration)."""
    config_dict = read_config_json(folder)
    arch = architecture_for(config_dict)
    config = arch.read_config(config_dict)
    return _build(arch.model_spec(config), FolderSource(folder), dtype, device), config


def random_model(config_dict: Dict[str, Any], seed: int, dtype="bfloat16", device="cuda:0",
                 weight_dtype: Optional[torch.dtype] = None, std: Optional[float] = None):
    """A model with random weights made in memory (on ``device``), without a folder."""
    arch = architecture_for(config_dict)
    config = arch.read_config(config_dict)
    spec = arch.model_spec(config)
    wdtype = weight_dtype or parse_dtype(dtype)
    tensors = dict(random_tensors(declared_tensors(spec), seed,
                                  spec.init_std if std is None else std, wdtype, device=str(device)))
    return _build(spec, DictSource(tensors, "<random weights>"), dtype, device), config
