"""What a mixer asks of the cache: pages of keys and values, or a fixed-size state per request.

The reference has one shape of cache for every layer (src/qwen.cc:507-516) and no per-request
state; here every site of the run order states its need and the manager groups equal needs.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch


@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every token, in pages.  ``window``: only the last ``window``
    positions are ever read again, so pages that lie wholly before them are given back."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class FixedState:
    """A tensor of fixed shape per live request (kept in a slot, zeroed when a request starts)."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32
