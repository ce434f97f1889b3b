"""A decoder-only language model assembled from a :class:`ModelSpec`: embedding, the layers in
their run order, final norm and output head.  It is the same class for every architecture; an
architecture only supplies the spec (see :mod:`lucciola_amd.models.qwen3`).

The forward pass follows the reference's step (src/qwen.cc:801-902: embedding -> layers ->
final norm -> head) with two differences of substance: the final norm and the head run only on
the rows whose logits are wanted (the reference norms all rows, src/qwen.cc:851-858), and the
logits leave as float32 (the reference keeps bf16 logits on the device and returns only the
argmax, src/qwen.cc:875-892).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..config.registry import BLOCKS, FEED_FORWARDS, MIXERS, NORMS
from ..config.specs import LayerSpec, ModelSpec
from ..engine.batch import SiteView, StepBatch
from ..kernels import ops
from ..parts import BuildContext, ResidualStream, build_part
from ..weights.loader import ParamDecl, WeightSource, load_declared


class _LayerParts:
    def __init__(self, spec: LayerSpec):
        self.spec = spec
        self.mixer = build_part(MIXERS, spec.mixer)
        self.feed_forward = build_part(FEED_FORWARDS, spec.feed_forward)
        self.mixer_norm = build_part(NORMS, spec.mixer_norm)
        self.feed_forward_norm = build_part(NORMS, spec.feed_forward_norm)
        self.block = BLOCKS.get(spec.block)(self.mixer, self.feed_forward, self.mixer_norm,
                                            self.feed_forward_norm)

    def parts(self):
        return (("mixer", self.mixer), ("feed_forward", self.feed_forward),
                ("mixer_norm", self.mixer_norm), ("feed_forward_norm", self.feed_forward_norm))

    def declared(self) -> Dict[str, ParamDecl]:
        """Checkpoint name -> declaration, through the layer's name map."""
        out: Dict[str, ParamDecl] = {}
        for prefix, part in self.parts():
            for logical, decl in part.declare().items():
                key = f"{prefix}.{logical}"
                if key not in self.spec.names:
                    raise KeyError(f"layer spec has no checkpoint name for '{key}'")
                out[self.spec.names[key]] = decl
        return out

    def bind(self, tensors: Dict[str, torch.Tensor], ctx: BuildContext) -> None:
        for prefix, part in self.parts():
            mine = {logical: tensors[self.spec.names[f"{prefix}.{logical}"]]
                    for logical in part.declare()}
            part.bind(mine, ctx)


def declared_tensors(spec: ModelSpec) -> Dict[str, ParamDecl]:
    """Every tensor a model of this spec wants, by checkpoint name."""
    spec.validate()
    out: Dict[str, ParamDecl] = {
        spec.embedding_name: ParamDecl((spec.vocab_size, spec.hidden_size))}
    for layer in spec.layers:
        out.update(_LayerParts(layer).declared())
    norm = build_part(NORMS, spec.final_norm)
    for logical, decl in norm.declare().items():
        out[spec.final_norm_names[logical]] = decl
    if spec.head_name is not None:
        out[spec.head_name] = ParamDecl((spec.vocab_size, spec.hidden_size))
    return out


class CausalLM:
    def __init__(self, spec: ModelSpec, source: WeightSource, dtype: torch.dtype, device,
                 optional_names=()):
        spec.validate()
        self.spec = spec
        self.ctx = BuildContext(dtype=dtype, device=torch.device(device))
        tensors = load_declared(source, declared_tensors(spec), self.ctx.device,
                                optional=optional_names)
        self.embedding = tensors[spec.embedding_name]
        self.head = tensors[spec.head_name] if spec.head_name is not None else self.embedding
        self.layers: List[_LayerParts] = []
        for layer_spec in spec.layers:
            layer = _LayerParts(layer_spec)
            layer.bind(tensors, self.ctx)
            self.layers.append(layer)
        self.final_norm = build_part(NORMS, spec.final_norm)
        self.final_norm.bind({logical: tensors[name]
                              for logical, name in spec.final_norm_names.items()}, self.ctx)
        self.vocab_size, self.hidden_size = spec.vocab_size, spec.hidden_size

    # ------------------------------------------------------------------ cache needs
    def site_needs(self) -> List[Optional[object]]:
        """For each site of the run order: what it needs of the cache (None when it reads
        another site's cache or needs nothing)."""
        needs = []
        for entry in self.spec.run_order:
            needs.append(None if entry.cache_of is not None
                         else self.layers[entry.layer].mixer.cache_need())
        return needs

    def graph_safe(self) -> bool:
        """Whether every part of every layer may be captured in a HIP graph."""
        return all(getattr(part, "graph_safe", False)
                   for layer in self.layers for _, part in layer.parts()) \
            and getattr(self.final_norm, "graph_safe", False)

    # ------------------------------------------------------------------ position tables
    def _position_parts(self):
        for layer in self.layers:
            pos = getattr(layer.mixer, "position", None)
            if pos is not None and hasattr(pos, "generation"):
                yield pos

    def position_epoch(self) -> int:
        """Changes whenever a position table has been made anew (its address has changed)."""
        return sum(p.generation for p in self._position_parts())

    def positions_ready(self, position: int) -> bool:
        """Whether every position table already covers ``position``."""
        return all(p.capacity() > position for p in self._position_parts())

    # ------------------------------------------------------------------ forward
    def forward(self, batch: StepBatch, sites: List[SiteView]) -> torch.Tensor:
        """Run the batch's tokens through every site; float32 logits [wanted, vocab]."""
        stream = ResidualStream(ops.embedding(batch.token_ids, self.embedding))
        for index, entry in enumerate(self.spec.run_order):
            self.layers[entry.layer].block.forward(stream, sites[index])
        if batch.num_wanted == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.ctx.device)
        x = self.final_norm.add_norm_rows(stream, batch.want_rows)
        return ops.gemm(x, self.head, torch.float32)
