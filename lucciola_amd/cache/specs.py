"""What a part asks of the cache: a *need*.  A need is an object that knows what it costs, how
its device memory is laid out and what a site gets to see of it; the cache manager only counts
pages and slots and never looks inside.

Two families are told apart by ``paged``.  A paged need grows with a request's tokens: the
manager keeps a pool of page ids and a block table per request for every group of equal needs,
and gives pages back when a request ends or a window has passed them.  A fixed need is one
piece of memory per live request, addressed by the request's slot.  Another layout of cache
(one latent tensor per token instead of a key/value pair, a ring of states, ...) is another
subclass of :class:`CacheNeed`; nothing else changes.

The reference has one shape of cache for every layer (src/qwen.cc:507-516) and no per-request
state.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional, Tuple

import torch


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


@dataclass(frozen=True)
class CacheLayout:
    """What the manager tells a need when its memory is made."""

    num_pages: int      # pages of the pool, in the manager's own pages
    page_size: int      # tokens of one of those pages
    kernel_page: int    # tokens of a page as the need's kernels index it (divides page_size)
    max_seqs: int       # live requests at most: the number of slots

    @property
    def kernel_pages(self) -> int:
        return self.num_pages * (self.page_size // self.kernel_page)


class CacheNeed:
    """Base of all needs.  Needs are compared with ``==`` and hashed: equal paged needs share
    one pool of pages and one block table per request (each site still has memory of its own).

    ``allocate`` returns whatever the part wants to find as ``site.cache``: a tensor, a tuple of
    tensors, an object of its own."""

    paged = False
    window: Optional[int] = None    # paged: only the last ``window`` positions are read again

    def kernel_page(self, page_size: int) -> int:
        """Tokens of a page as this need's kernels index it, for the manager's page size: a
        divisor of ``page_size``.  Where it is smaller, a page lies in memory as that many
        kernel pages in a row and the block tables that reach the device name those."""
        return page_size

    def bytes_per_page(self, page_size: int, dtype: torch.dtype) -> int:
        """Paged needs: bytes of one page of ``page_size`` tokens at one site."""
        return 0

    def bytes_per_request(self, dtype: torch.dtype) -> int:
        """Fixed needs: bytes of one request's piece at one site."""
        return 0

    def allocate(self, layout: CacheLayout, dtype: torch.dtype, device) -> Any:
        raise NotImplementedError

    def start(self, storage: Any, slot: int) -> None:
        """A request begins in ``slot``: bring what it will find there to its initial state."""


@dataclass(frozen=True)
class PagedKV(CacheNeed):
    """Keys and values of every token, in pages.  ``window``: only the last ``window``
    positions are ever read again, so pages that lie wholly before them are given back.
    ``granule``: the page size the part's kernels are built for; a page of a multiple of it is
    handed to them as so many pages of that size.

    Memory per site: keys ``[pages, kv_heads, page, head_dim]`` and values ``[pages, kv_heads,
    head_dim, page]`` (transposed inside a page), in kernel pages."""

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    granule: Optional[int] = None

    paged = True

    def kernel_page(self, page_size: int) -> int:
        g = self.granule
        return g if g and page_size > g and page_size % g == 0 else page_size

    def bytes_per_page(self, page_size: int, dtype: torch.dtype) -> int:
        return 2 * self.num_kv_heads * page_size * self.head_dim * _element_size(dtype)

    def allocate(self, layout: CacheLayout, dtype: torch.dtype, device):
        pages, page = layout.kernel_pages, layout.kernel_page
        keys = torch.zeros((pages, self.num_kv_heads, page, self.head_dim), dtype=dtype, device=device)
        values = torch.zeros((pages, self.num_kv_heads, self.head_dim, page), dtype=dtype, device=device)
        return keys, values


@dataclass(frozen=True)
class FixedState(CacheNeed):
    """A tensor of fixed shape per live request: ``[max_seqs, *shape]``, indexed by the
    request's slot and zeroed when a request starts."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def bytes_per_request(self, dtype: torch.dtype) -> int:
        count = 1
        for n in self.shape:
            count *= int(n)
        return count * _element_size(self.dtype)

    def allocate(self, layout: CacheLayout, dtype: torch.dtype, device):
        return torch.zeros((layout.max_seqs,) + tuple(self.shape), dtype=self.dtype, device=device)

    def start(self, storage, slot: int) -> None:
        storage[slot].zero_()
