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

import math
import sys
from typing import Callable, Dict, List, Optional

import torch

from ..config.registry import BLOCKS, EMBEDDINGS, FAMILIES, HEADS, NORMS
from ..config.specs import LayerSpec, ModelSpec, PartSpec
from ..engine.batch import SiteView, StepBatch
from ..parts import BuildContext, ResidualStream, build_part
from ..weights.loader import ParamDecl, WeightSource, load_declared, precision_notices


class _LayerParts:
    """The parts of one layer, built from its spec, and the block that arranges them."""

    def __init__(self, spec: LayerSpec):
        self.spec = spec
        block_cls = BLOCKS.get(spec.block)
        slots = getattr(block_cls, "slots", None)
        if not isinstance(slots, dict):
            raise TypeError(f"block arrangement '{spec.block}' does not say which slots it has")
        if set(slots) != set(spec.parts):
            raise ValueError(f"block arrangement '{spec.block}' has the slots {sorted(slots)}, "
                             f"the layer gives {sorted(spec.parts)}")
        self.by_slot = {}
        for slot, family in slots.items():
            if family not in FAMILIES:
                raise ValueError(f"block arrangement '{spec.block}': slot '{slot}' names the "
                                 f"unknown family '{family}'")
            self.by_slot[slot] = build_part(FAMILIES[family], spec.parts[slot])
        self.block = block_cls(**self.by_slot)
        # the parts that keep something in the cache, in the order of the block's slots: a site's
        # view holds their memory in this order (``SiteView.caches``, ``SiteView.part(k)``)
        self.caching = [p for p in self.by_slot.values() if p.cache_need() is not None]

    def __getattr__(self, slot):          # layer.mixer, layer.feed_forward_norm, ...
        try:
            return self.__dict__["by_slot"][slot]
        except KeyError:
            raise AttributeError(slot) from None

    def parts(self):
        return tuple(self.by_slot.items())

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


def _end_parts(spec: ModelSpec):
    """The embedding and the head of a spec (built, not bound) and the head's name map."""
    sizes = {"vocab_size": spec.vocab_size, "hidden_size": spec.hidden_size}
    embedding = build_part(EMBEDDINGS, spec.embedding or PartSpec("token_embedding", sizes))
    head_spec = spec.head or PartSpec("linear_head", sizes)
    head = build_part(HEADS, head_spec.with_params(tied=spec.head_name is None))
    head_names = dict(spec.head_names or {})
    if spec.head_name is not None:
        head_names.setdefault("weight", spec.head_name)
    return embedding, head, head_names


def declared_tensors(spec: ModelSpec) -> Dict[str, ParamDecl]:
    """Every tensor a model of this spec wants, by checkpoint name."""
    spec.validate()
    embedding, head, head_names = _end_parts(spec)
    out: Dict[str, ParamDecl] = {}
    for logical, decl in embedding.declare().items():
        if logical != "weight":
            raise KeyError(f"the embedding's tensor '{logical}' has no checkpoint name")
        out[spec.embedding_name] = decl
    for layer in spec.layers:
        out.update(_LayerParts(layer).declared())
    norm = build_part(NORMS, spec.final_norm)
    for logical, decl in norm.declare().items():
        out[spec.final_norm_names[logical]] = decl
    for logical, decl in head.declare().items():
        if logical not in head_names:
            raise KeyError(f"the head's tensor '{logical}' has no checkpoint name")
        out[head_names[logical]] = decl
    return out


class CausalLM:
    def __init__(self, spec: ModelSpec, source: WeightSource, dtype: torch.dtype, device,
                 optional_names=()):
        spec.validate()
        self.spec = spec
        self.ctx = BuildContext(dtype=dtype, device=torch.device(device))
        declared = declared_tensors(spec)
        stored: Dict[str, torch.dtype] = {}
        tensors = load_declared(source, declared, self.ctx.device, optional=optional_names,
                                stored_dtypes=stored)
        # what the kept dtypes cost, said once per class of tensor
        self.load_notices = precision_notices(stored, declared, self.ctx.dtype)
        for line in self.load_notices:
            print(f"[lucciola_amd] {line}", file=sys.stderr, flush=True)
        self.embed, self.head_part, head_names = _end_parts(spec)
        self.embed.bind({"weight": tensors[spec.embedding_name]}, self.ctx)
        self.head_part.bind({logical: tensors[head_names[logical]]
                             for logical in self.head_part.declare()}, self.ctx,
                            shared=self.embed.table())
        self.layers: List[_LayerParts] = []
        for layer_spec in spec.layers:
            layer = _LayerParts(layer_spec)
            layer.bind(tensors, self.ctx)
            self.layers.append(layer)
        self.final_norm = build_part(NORMS, spec.final_norm)
        self.final_norm.bind({logical: tensors[name]
                              for logical, name in spec.final_norm_names.items()}, self.ctx)
        self.vocab_size, self.hidden_size = spec.vocab_size, spec.hidden_size

    @property
    def embedding(self) -> torch.Tensor:
        return self.embed.table()

    @property
    def head(self) -> torch.Tensor:
        return self.head_part.weight

    def _all_parts(self):
        for layer in self.layers:
            for _, part in layer.parts():
                yield part

    # ------------------------------------------------------------------ cache needs
    def site_needs(self) -> List[Optional[object]]:
        """For each site of the run order: what it needs of the cache: a need, a tuple of needs
        (a layer with several caching parts) or None (it reads another site's cache or needs
        nothing)."""
        needs = []
        for entry in self.spec.run_order:
            caching = self.layers[entry.layer].caching
            if entry.cache_of is not None or not caching:
                needs.append(None)
            else:
                mine = tuple(part.cache_need() for part in caching)
                needs.append(mine[0] if len(mine) == 1 else mine)
        return needs

    def graph_safe(self) -> bool:
        """Whether every part may be captured in a HIP graph."""
        return all(getattr(part, "graph_safe", False) for part in self._all_parts()) \
            and all(getattr(p, "graph_safe", False) for p in (self.final_norm, self.embed, self.head_part))

    def batch_planners(self) -> Dict[object, Callable]:
        """The work lists that parts want made from every step's batch (``Part.batch_planner``),
        one per distinct key."""
        planners: Dict[object, Callable] = {}
        for part in self._all_parts():
            planner = part.batch_planner()
            if planner is not None:
                planners.setdefault(planner[0], planner[1])
        return planners

    def portion_multiple(self) -> int:
        """Portions of a prompt, but for its last, must be multiples of this many tokens."""
        multiple = 1
        for part in self._all_parts():
            multiple = math.lcm(multiple, int(getattr(part, "portion_multiple", 1)))
        return multiple

    # ------------------------------------------------------------------ tables that parts grow
    def tables_epoch(self) -> int:
        """Changes whenever a part has made a device table anew (``Part.tables_epoch``): kernel
        arguments captured before that point at the old one."""
        return sum(part.tables_epoch() for part in self._all_parts())

    def ready(self, position: int) -> bool:
        """Whether every part can serve ``position`` without making a table anew."""
        return all(part.ready(position) for part in self._all_parts())

    # ------------------------------------------------------------------ forward
    def forward(self, batch: StepBatch, sites: List[SiteView]) -> torch.Tensor:
        """Run the batch's tokens through every site; float32 logits [wanted, vocab]."""
        stream = ResidualStream(self.embed.forward(batch.token_ids))
        for index, entry in enumerate(self.spec.run_order):
            self.layers[entry.layer].block.forward(stream, sites[index])
        if batch.num_wanted == 0:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.ctx.device)
        x = self.final_norm.add_norm_rows(stream, batch.want_rows)
        return self.head_part.forward(x)
