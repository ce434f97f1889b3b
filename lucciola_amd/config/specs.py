"""Data that describes a model: which parts each layer is made of, and the order in which
layers run.  Nothing in here knows an architecture; an architecture's builder fills these
records from its typed configuration and the generic model is assembled from them.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: the registered kind and the sizes/constants it is built with."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def with_params(self, **more: Any) -> "PartSpec":
        merged = dict(self.params)
        merged.update(more)
        return PartSpec(self.kind, merged)


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: a block arrangement and the parts that fill its slots.

    The block kind decides which slots there are and of which family each is (its ``slots``:
    the pre-norm residual block has a mixer, a feed-forward and a norm before each; another
    arrangement may have one shared norm, or no feed-forward).  ``names`` maps each part's
    logical tensor name, prefixed with its slot (``"mixer.q_proj"``), to the name the
    checkpoint uses (``"model.layers.3.self_attn.q_proj.weight"``).
    """

    block: str
    parts: Dict[str, PartSpec]
    names: Dict[str, str]


def prenorm_layer(mixer: PartSpec, feed_forward: PartSpec, mixer_norm: PartSpec,
                  feed_forward_norm: PartSpec, names: Dict[str, str]) -> LayerSpec:
    """A layer in the pre-norm residual arrangement (``prenorm_residual``)."""
    return LayerSpec("prenorm_residual",
                     {"mixer": mixer, "feed_forward": feed_forward, "mixer_norm": mixer_norm,
                      "feed_forward_norm": feed_forward_norm}, names)


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order: run ``layer`` here.

    A layer may be named by several entries; each entry is a *site* with a cache of its own.
    ``cache_of`` names an earlier site whose cache this site reads instead of writing one.
    """

    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding_name: str
    layers: List[LayerSpec]
    run_order: List[RunEntry]
    final_norm: PartSpec
    final_norm_names: Dict[str, str]
    head_name: Optional[str]  # None: the head uses the embedding table (tied)
    init_std: float = 0.02
    max_positions: int = 0  # 0: no guard
    # the parts at the model's two ends; None: a plain table look-up and a plain bias-free
    # product, built from vocab_size and hidden_size
    embedding: Optional[PartSpec] = None
    head: Optional[PartSpec] = None
    head_names: Optional[Dict[str, str]] = None   # a head with tensors beyond "weight" names them here

    def validate(self) -> None:
        for i, entry in enumerate(self.run_order):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"run_order[{i}] names layer {entry.layer}, "
                                 f"but there are {len(self.layers)} layers")
            if entry.cache_of is not None:
                if not 0 <= entry.cache_of < i:
                    raise ValueError(f"run_order[{i}].cache_of={entry.cache_of} must name an "
                                     f"earlier site")
                if self.run_order[entry.cache_of].cache_of is not None:
                    raise ValueError(f"run_order[{i}].cache_of={entry.cache_of} names a site "
                                     f"that itself has no cache of its own")
