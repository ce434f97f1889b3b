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
    """One decoder layer: an arrangement (block kind) of a mixer, a feed-forward and norms.

    ``names`` maps each part's logical tensor name (``"mixer.q_proj"``) to the name the
    checkpoint uses (``"model.layers.3.self_attn.q_proj.weight"``).
    """

    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    names: Dict[str, str]


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
