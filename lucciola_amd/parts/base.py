"""What every part of a layer has in common, and the residual stream that blocks pass along.

A part is built from its sizes and constants alone (``PartSpec.params``), declares the tensors
it wants under logical names, and gets them in ``bind``.  No part knows which model it is in
or what the checkpoint calls its tensors: the architecture maps logical names to checkpoint
names (``LayerSpec.names``).

Interfaces (all tensors on the GPU; "act" is the engine's activation dtype):
  Norm            add_norm(stream) -> act [T, n]; add_norm_rows(stream, rows) -> act [R, n];
                  fused_rms() -> (weight float32 [n], eps) or None.  A norm with
                  offers_scaled_rows = True also has add_norm(stream, scaled=True), which may
                  return ops.ScaledRows; stream.pending may be an ops.PendingProduct
  PositionEncoding  rotary_table(max_position) -> float32 [positions, rot] or None;
                  apply(qkv, nh, nkv, d, positions) in place, when there is no table
  Mixer           forward(x act [T, H], site: SiteView) -> act [T, H]; cache_need() -> a
                  CacheNeed or None; batch_planner() -> (key, plan) or None; portion_multiple;
                  tables_epoch(), ready(position) where it grows device tables
  FeedForward     forward(x act [T, H]) -> act [T, H]
                  A mixer or feed-forward with takes_scaled_rows = True may be given
                  ops.ScaledRows as x (ops.gemm and ops.gemm_swiglu take them) and may return
                  ops.gemm(..., defer=True); ops.value(t) turns either into a tensor
  Block           slots = {slot name: family}; built with the layer's parts by slot name;
                  forward(stream, site) -> None (updates the stream)
  Embedding, Head the model's two ends (parts/ends.py)
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict

import torch

from ..config.registry import Registry
from ..config.specs import PartSpec
from ..weights.loader import ParamDecl


@dataclass
class BuildContext:
    dtype: torch.dtype      # activation dtype of the engine: bfloat16 or float32
    device: torch.device
    # what parts of ONE model share (a position table that all its layers use): made with the
    # model, gone with it; nothing is shared between models
    shared: Dict[Any, Any] = field(default_factory=dict)


class ResidualStream:
    """The float32 residual stream ``h`` [T, H] and the branch output that is still to be added.

    The sum h + pending is formed in float32 inside the next norm's kernel (the reference adds
    in float32 and rounds the stream to bf16, src/kernels/add.cu:11-14; here the stream itself
    stays float32)."""

    def __init__(self, h: torch.Tensor):
        self.h = h
        self.pending = None      # a tensor [T, H] or an ops.PendingProduct


class Part:
    """Base of all parts.  A part is built from keyword parameters (its sizes and constants)."""

    # True if ``forward`` only launches kernels on tensors whose addresses and shapes depend
    # on nothing but the batch layout (no host-side reads of batch values, no loops over
    # requests): such a part may be captured in a HIP graph and replayed.  A captured step of
    # five or more requests is filled up with copies of its first entry (same token, same
    # position, same pages), so what such a part writes for a request must be the same when
    # written twice; a model with per-request state slots is never filled up this way.
    graph_safe = False

    # Portions of a prompt, but for its last, are cut at multiples of this many tokens (a
    # mixer whose kernel works on whole blocks of tokens sets it; the scheduler obeys it).
    portion_multiple = 1

    def __init__(self, **params: Any):
        self.params = dict(params)

    def declare(self) -> Dict[str, ParamDecl]:
        """Logical tensor name -> declaration."""
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], ctx: BuildContext) -> None:
        """Take the declared tensors (already on the device, in their kept dtype)."""

    def cache_need(self):
        """What this part keeps in the cache: a ``cache.specs.CacheNeed`` (PagedKV, FixedState or
        a subclass of the part's own) or None.  What the need allocates is what the part finds
        as ``site.cache``; a paged need also finds ``site.pages`` (block table, slots, page
        size)."""
        return None

    def tables_epoch(self) -> int:
        """A number that changes whenever this part has made a device table anew whose address
        kernels take as an argument (a position table that has grown): steps captured before
        are captured again.  A part that nests other parts adds theirs."""
        return 0

    def ready(self, position: int) -> bool:
        """Whether the part can serve ``position`` without making such a table anew."""
        return True

    def batch_planner(self):
        """Work lists this part's kernels want made from every step's batch, once a step and
        not once a layer: ``(key, plan)`` or None.  ``plan(layout: engine.batch.HostLayout)``
        returns ``(arrays, info)``: named int32 arrays (numpy), which reach the GPU in the
        batch's one copy, and host-side numbers.  Parts with equal keys share one plan; the
        part finds it as ``site.batch.plans[key]`` (``.arrays`` on the device, ``.info``).
        For batches of the same make-up the arrays must have the same sizes (captured steps
        refresh them in place).  Where a kernel's launch depends on more of the batch than its
        make-up, ``info["graph_hint"]`` (hashable) names the class of batches that share a
        launch: a captured step is replayed only for batches of its own hint."""
        return None


def build_part(registry: Registry, spec: PartSpec) -> Part:
    cls = registry.get(spec.kind)
    return cls(**spec.params)


def require(params: Dict[str, Any], *keys: str, part: str) -> None:
    missing = [k for k in keys if k not in params]
    if missing:
        raise TypeError(f"{part}: missing parameters {missing}")
