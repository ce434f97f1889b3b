"""RMSNorm as a part: ``y = x * rsqrt(mean(x^2) + eps) * w`` over the last dimension
(reference: src/kernels/rmsnorm.cu:56-97; eps is the literal 1e-6 there, src/qwen.cc:588, and
a parameter here)."""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from ..config.registry import NORMS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, ResidualStream


@NORMS.register("rms")
class RMSNorm(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps
    offers_scaled_rows = True   # add_norm(stream, scaled=True) may return ops.ScaledRows

    def __init__(self, size: int, eps: float):
        super().__init__(size=size, eps=eps)
        self.size, self.eps = int(size), float(eps)
        self.weight: Optional[torch.Tensor] = None
        self.dtype = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.size,), role="vector", init="ones_plus_normal")}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.weight = tensors["weight"]
        self.dtype = ctx.dtype

    def add_norm(self, stream: ResidualStream, scaled: bool = False):
        """Add the pending branch output into the stream and return the normed stream
        (``scaled``: the caller also takes ops.ScaledRows)."""
        x = ops.rmsnorm(stream.h, stream.pending, self.weight, self.eps, self.dtype, scaled=scaled)
        stream.pending = None
        return x

    def add_norm_rows(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        """The normed stream (pending included) at the given rows only; the stream is not changed."""
        return ops.rmsnorm(stream.h, stream.pending, self.weight, self.eps, self.dtype, rows=rows)

    def apply(self, x: torch.Tensor) -> torch.Tensor:
        """Norm over the last dimension of an activation tensor."""
        return ops.rmsnorm_act(x, self.weight, self.eps)

    def fused_rms(self) -> Optional[Tuple[torch.Tensor, float]]:
        return self.weight, self.eps
