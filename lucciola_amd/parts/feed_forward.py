"""The gated feed-forward (SwiGLU) as a part: ``down(silu(gate(x)) * up(x))``, no biases
(reference: src/qwen.cc:762-794, src/kernels/swiglu.cu:8,31-35).  gate and up are one matrix
product here: their weights are stacked at load."""
from __future__ import annotations

from typing import Dict

import torch

from ..config.registry import FEED_FORWARDS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part


def stack_rows(tensors):
    """Stack weight matrices along their rows; mixed storage widens to float32."""
    dtypes = {t.dtype for t in tensors}
    if len(dtypes) > 1:
        tensors = [t.to(torch.float32) for t in tensors]
    return torch.cat(tensors, dim=0).contiguous()


@FEED_FORWARDS.register("gated_mlp")
class GatedMLP(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps
    takes_scaled_rows = True   # x may be ops.ScaledRows; the output may be an ops.PendingProduct

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        super().__init__(hidden_size=hidden_size, intermediate_size=intermediate_size,
                         activation=activation)
        if activation != "silu":
            raise ValueError(f"gated_mlp: activation '{activation}' has no kernel (only silu)")
        self.H, self.I = int(hidden_size), int(intermediate_size)

    def declare(self) -> Dict[str, ParamDecl]:
        return {"gate_proj": ParamDecl((self.I, self.H)),
                "up_proj": ParamDecl((self.I, self.H)),
                "down_proj": ParamDecl((self.H, self.I))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        gate, up = tensors["gate_proj"], tensors["up_proj"]
        self.down = tensors["down_proj"]
        self.dtype = ctx.dtype
        # where the matrix-core kernel takes the sizes, gate and up rows are interleaved so that
        # silu(gate) * up is formed in the product's epilogue and [T, 2 I] never reaches memory
        self.fused = (ctx.device.type == "cuda" and self.I % 8 == 0 and gate.dtype == up.dtype
                      and ops.gemm_swiglu_supported(ctx.dtype, gate.new_empty((2 * self.I, 1)), self.H))
        if self.fused:
            self.gate_up = ops.interleave_gate_up(gate, up)
        else:
            self.gate_up = stack_rows([gate, up])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self.fused:
            z = ops.gemm_swiglu(x, self.gate_up)
        else:
            z = ops.swiglu(ops.gemm(x, self.gate_up, self.dtype))
        return ops.gemm(z, self.down, self.dtype, defer=True)
