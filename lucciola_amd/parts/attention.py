"""Grouped-query attention over the paged cache, as a part.

Order of operations as in the reference's layer (src/qwen.cc:592-738): q, k, v projections
(one product here, the weights are stacked at load) -> RMSNorm over head_dim on every q and k
head with one [d] weight each -> rotary embedding of q and k -> k, v written to the cache ->
causal attention over all cached keys (kv head = h / (nh / nkv), scale 1/sqrt(d)) -> output
projection.  Sizes, the scale, the norm, the position encoding and an optional window are
parameters; nh * d need not equal the hidden size.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..cache.specs import PagedKV
from ..config.registry import MIXERS, NORMS, POSITION_ENCODINGS
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.loader import ParamDecl
from .base import BuildContext, Part, build_part
from .feed_forward import stack_rows


@MIXERS.register("attention")
class Attention(Part):
    graph_safe = True   # launches only kernels whose arguments stay put between steps
    takes_scaled_rows = True   # x may be ops.ScaledRows; the output may be an ops.PendingProduct

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: Optional[float] = None, qk_norm: Optional[PartSpec] = None,
                 position: Optional[PartSpec] = None, window: Optional[int] = None):
        super().__init__(hidden_size=hidden_size, num_heads=num_heads, num_kv_heads=num_kv_heads,
                         head_dim=head_dim, scale=scale, qk_norm=qk_norm, position=position,
                         window=window)
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of "
                             f"{num_kv_heads} kv heads")
        self.H, self.nh, self.nkv, self.d = int(hidden_size), int(num_heads), int(num_kv_heads), int(head_dim)
        self.scale = float(scale) if scale is not None else self.d ** -0.5
        self.window = int(window) if window else None
        self.fused_qk_norm = True
        self.q_norm = build_part(NORMS, qk_norm) if qk_norm else None
        self.k_norm = build_part(NORMS, qk_norm) if qk_norm else None
        self.position = build_part(POSITION_ENCODINGS, position) if position else None

    def declare(self) -> Dict[str, ParamDecl]:
        out = {"q_proj": ParamDecl((self.nh * self.d, self.H)),
               "k_proj": ParamDecl((self.nkv * self.d, self.H)),
               "v_proj": ParamDecl((self.nkv * self.d, self.H)),
               "o_proj": ParamDecl((self.H, self.nh * self.d))}
        if self.q_norm is not None:
            for name, decl in self.q_norm.declare().items():
                out["q_norm." + name] = decl
            for name, decl in self.k_norm.declare().items():
                out["k_norm." + name] = decl
        return out

    def bind(self, tensors, ctx: BuildContext) -> None:
        self.qkv = stack_rows([tensors["q_proj"], tensors["k_proj"], tensors["v_proj"]])
        self.o = tensors["o_proj"]
        self.dtype = ctx.dtype
        if self.q_norm is not None:
            self.q_norm.bind({k[7:]: v for k, v in tensors.items() if k.startswith("q_norm.")}, ctx)
            self.k_norm.bind({k[7:]: v for k, v in tensors.items() if k.startswith("k_norm.")}, ctx)
            # a norm that the fused kernel cannot apply (no fused_rms()) is applied through its
            # own ``apply`` on the heads, one kernel more a step
            fused = getattr(self.q_norm, "fused_rms", None)
            self.fused_qk_norm = fused is not None and fused() is not None
            if not self.fused_qk_norm and not hasattr(self.q_norm, "apply"):
                raise NotImplementedError("attention: the q/k norm must offer fused_rms() or apply()")
        if self.position is not None:
            self.position.bind({}, ctx)

    def _norm_heads(self, qkv: torch.Tensor) -> None:
        """The q and k heads of ``qkv`` [T, (nh + 2 nkv) d] through the norms' own ``apply``."""
        T = qkv.shape[0]
        for norm, first, heads in ((self.q_norm, 0, self.nh), (self.k_norm, self.nh, self.nkv)):
            cols = slice(first * self.d, (first + heads) * self.d)
            x = qkv[:, cols].contiguous().view(T * heads, self.d)
            qkv[:, cols] = norm.apply(x).view(T, heads * self.d)

    def cache_need(self):
        return PagedKV(self.nkv, self.d, self.window, granule=ops.attention_page_granule())

    def batch_planner(self):
        return ops.ATTENTION_PLAN, ops.plan_attention

    def tables_epoch(self) -> int:
        return self.position.tables_epoch() if self.position is not None else 0

    def ready(self, position: int) -> bool:
        return self.position.ready(position) if self.position is not None else True

    def forward(self, x: torch.Tensor, site) -> torch.Tensor:
        # the attention kernels' record of the step: made once a step for the page group, from
        # the batch, the group's pages and the work lists of this part's planner
        attn = ops.attention_batch(site.batch, site.pages, site.batch.plans.get(ops.ATTENTION_PLAN))
        page_size = site.pages.page_size
        q_w = k_w = None
        eps = 0.0
        own_norm = self.q_norm is not None and not self.fused_qk_norm
        if self.q_norm is not None and self.fused_qk_norm:
            q_w, eps = self.q_norm.fused_rms()
            k_w, _ = self.k_norm.fused_rms()
        table = None
        if self.position is not None:
            table = self.position.rotary_table(site.batch.max_position)
        # where the q/k/v product is cut along K and the attention kernel can sum its shares
        # as it reads them, the kernel that would sum them is saved
        rows = x.x.shape[0] if isinstance(x, ops.ScaledRows) else x.shape[0]
        as_shares = ((table is not None or self.position is None) and not own_norm
                     and ops.attention_takes_shares(attn, rows, self.nh, self.nkv, self.d, page_size,
                                                    self.dtype, table.shape[1] if table is not None else 0))
        qkv = ops.gemm(x, self.qkv, self.dtype, shares=as_shares)
        if own_norm:
            self._norm_heads(qkv)
        if self.position is not None and table is None:
            self.position.apply(qkv, self.nh, self.nkv, self.d, attn.positions)
        k_cache, v_cache = site.cache
        prologue = ops.QKPrologue(q_w, k_w, eps, table, attn.slots if site.writes_cache else None)
        o = ops.attention(qkv, attn, k_cache, v_cache, self.nh, self.nkv, self.d, page_size,
                          self.scale, self.window or 0, prologue)
        return ops.gemm(o, self.o, self.dtype, defer=True)
