"""The parts at a model's two ends: the token embedding, which starts the float32 residual
stream, and the output head, which turns normed rows into float32 logits.

The reference gathers rows of ``model.embed_tokens.weight`` (src/qwen.cc:830-837,
src/kernels/embedding.cu:22-38) and multiplies the normed last rows by ``lm_head.weight``, or by
the embedding table again when the checkpoint has no head (src/qwen.cc:80-84,875-882).  They are
parts like any other, so that an architecture with a scaled embedding, a head with a bias or
capped logits registers its own kind and the model class stays as it is.

Interfaces:
  Embedding   declare() -> {"weight": ...}; forward(ids int32 [T]) -> float32 [T, H];
              table() -> the tensor a tied head shares
  Head        declare() (nothing when tied); bind(tensors, ctx, shared=table or None);
              forward(x act [R, H]) -> float32 [R, V]
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config.registry import EMBEDDINGS, HEADS
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part


@EMBEDDINGS.register("token_embedding")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0):
        super().__init__(vocab_size=vocab_size, hidden_size=hidden_size, scale=scale)
        self.V, self.H, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.weight: Optional[torch.Tensor] = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {"weight": ParamDecl((self.V, self.H))}

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.weight = tensors["weight"]

    def table(self) -> torch.Tensor:
        return self.weight

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return ops.embedding(ids, self.weight, self.scale)


@HEADS.register("linear_head")
class LinearHead(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False):
        super().__init__(vocab_size=vocab_size, hidden_size=hidden_size, tied=tied)
        self.V, self.H, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.weight: Optional[torch.Tensor] = None

    def declare(self) -> Dict[str, ParamDecl]:
        return {} if self.tied else {"weight": ParamDecl((self.V, self.H))}

    def bind(self, tensors, ctx: BuildContext, shared: Optional[torch.Tensor] = None) -> None:
        self.weight = shared if self.tied else tensors["weight"]
        if self.weight is None:
            raise ValueError("linear_head: a tied head needs the embedding's table")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.gemm(x, self.weight, torch.float32)
