"""Rotary position embedding as a part.

Half-split pairing as the reference computes it (src/kernels/rope.cu:28-60): for i in
[0, rot/2): angle = pos / theta^(2i/rot); (x[i], x[i + rot/2]) is rotated by that angle.
theta is the literal 1e6 in the reference (src/qwen.cc:636) and a parameter here.  The
angles' cosines and sines are tabulated once per position (computed in float64, stored as
float32) and the kernel looks them up; the table grows when a longer position shows up.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..config.registry import POSITION_ENCODINGS
from .base import BuildContext, Part


class _SharedTable:
    """One table for all parts of a model with the same rotated size and base (its layers,
    usually), kept in the model's ``BuildContext.shared``: ``generation`` counts how often it
    has been made anew."""

    def __init__(self) -> None:
        self.table: Optional[torch.Tensor] = None
        self.generation = 0


@POSITION_ENCODINGS.register("rotary")
class Rotary(Part):
    def __init__(self, rotary_dim: int, theta: float, max_positions: int = 0):
        super().__init__(rotary_dim=rotary_dim, theta=theta, max_positions=max_positions)
        if rotary_dim % 2:
            raise ValueError(f"rotary: the rotated size {rotary_dim} must be even")
        self.rotary_dim, self.theta = int(rotary_dim), float(theta)
        self.initial = int(max_positions)
        self._shared = _SharedTable()
        self._device = None

    def bind(self, tensors, ctx: BuildContext) -> None:
        self._device = ctx.device
        self._shared = ctx.shared.setdefault(("rotary table", self.rotary_dim, self.theta), _SharedTable())

    def tables_epoch(self) -> int:
        return self._shared.generation

    def ready(self, position: int) -> bool:
        return self.capacity() > position

    @property
    def _table(self) -> Optional[torch.Tensor]:
        return self._shared.table

    def _make(self, count: int) -> torch.Tensor:
        half = self.rotary_dim // 2
        i = torch.arange(half, dtype=torch.float64)
        inv_freq = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64),
                                   2.0 * i / self.rotary_dim)
        angle = torch.arange(count, dtype=torch.float64)[:, None] * inv_freq[None, :]
        table = torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).to(torch.float32)
        return table.contiguous().to(self._device)

    def rotary_table(self, max_position: int) -> torch.Tensor:
        """float32 [positions, rot]: cosines in the first half of a row, sines in the second."""
        need = max_position + 1
        if self._table is None or self._table.shape[0] < need:
            count = max(need, min(self.initial, 16384), 256)
            if self._table is not None:
                count = max(count, 2 * self._table.shape[0])
            self._shared.table = self._make(count)
            self._shared.generation += 1
        return self._table

    def capacity(self) -> int:
        """Positions the present table covers."""
        return 0 if self._table is None else int(self._table.shape[0])

    def apply(self, qkv, nh, nkv, d, positions) -> None:  # the table path covers this part
        raise NotImplementedError
