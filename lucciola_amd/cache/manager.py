"""The cache manager: pages of keys and values with a block table per request, and slots for
per-request state of fixed size.

Every site of a model's run order states what it needs (:mod:`lucciola_amd.cache.specs`).
Sites with equal paged needs form a *group*: one pool of page ids and one block table per
request serve the whole group, and each site of the group has key and value tensors of its
own that are indexed by those page ids.  Groups differ in what they keep: all keys, or a
window of them, in which case the pages the window has passed are given back after each step.

The reference has one group (every layer alike, src/qwen.cc:507-516), takes a page when
``ceil(len / block_size)`` exceeds the table (src/scheduler.cc:55-58,89-97) and gives all of
a request's pages back when it ends (src/scheduler.cc:20-31).  The bookkeeping here is host
code only; the tensors are made by :meth:`CacheManager.allocate_tensors`.
"""
from __future__ import annotations

from array import array
from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from .page_pool import OutOfPages, PagePool, SlotPool
from .specs import FixedState, PagedKV


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


@dataclass
class PageGroup:
    spec: PagedKV
    sites: List[int]
    pool: PagePool
    # a request's page ids in order, as a typed array (numpy views it without a copy); -1: given back
    tables: Dict[Hashable, array] = field(default_factory=dict)


@dataclass
class RequestState:
    slot: int
    length: int = 0           # tokens whose keys/values (or state) are in the cache
    pending: int = 0          # tokens reserved by `reserve` and not yet committed
    started: bool = False     # False until the first commit: state slots are zeroed then


KERNEL_PAGE = 16       # tokens of a page as the kernels see it, where the page size is a multiple of it


class CacheManager:
    def __init__(self, site_specs: Sequence[Optional[object]], block_size: int, num_blocks: int,
                 max_seqs: int, scatter_pages: bool = True):
        """``site_specs[i]``: what site i of the run order needs (PagedKV, FixedState or None).
        A site that reads another site's cache is passed as None here.  ``scatter_pages``: see
        :class:`PagePool`."""
        if block_size <= 0 or num_blocks <= 0:
            raise ValueError("block_size and num_blocks must be positive")
        self.block_size = block_size
        # What the kernels see: a page of 32, 48, 64, ... tokens lies in memory as that many
        # pages of 16 in a row, each in the layout of a page of 16, and the block tables that
        # go to the device name those (page p becomes p * pieces ... p * pieces + pieces - 1).
        # A slot id, page * block_size + offset, is the same number either way.  So the
        # matrix-core kernels, which are built for pages of 16, serve every such size.
        self.kernel_block = KERNEL_PAGE if block_size > KERNEL_PAGE and block_size % KERNEL_PAGE == 0 \
            else block_size
        self.pieces = block_size // self.kernel_block
        self.num_blocks = num_blocks
        self.max_seqs = max_seqs
        self.site_specs = list(site_specs)
        self.groups: List[PageGroup] = []
        self.site_group: Dict[int, int] = {}
        self.state_sites: List[int] = []
        for i, spec in enumerate(self.site_specs):
            if spec is None:
                continue
            if isinstance(spec, PagedKV):
                for gi, g in enumerate(self.groups):
                    if g.spec == spec:
                        g.sites.append(i)
                        self.site_group[i] = gi
                        break
                else:
                    self.groups.append(PageGroup(spec, [i], PagePool(num_blocks, scatter_pages)))
                    self.site_group[i] = len(self.groups) - 1
            elif isinstance(spec, FixedState):
                self.state_sites.append(i)
            else:
                raise TypeError(f"site {i}: unknown cache need {spec!r}")
        self.slots = SlotPool(max_seqs)
        self.requests: Dict[Hashable, RequestState] = {}
        # device tensors (made by allocate_tensors)
        self.kv: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        self.state: Dict[int, torch.Tensor] = {}

    # ------------------------------------------------------------------ tensors
    def bytes_per_block(self, dtype: torch.dtype) -> int:
        size = torch.empty((), dtype=dtype).element_size()
        total = 0
        for g in self.groups:
            total += len(g.sites) * 2 * g.spec.num_kv_heads * self.block_size * g.spec.head_dim * size
        return total

    def state_bytes(self) -> int:
        """Bytes of the per-request state tensors of all state sites."""
        total = 0
        for site in self.state_sites:
            spec = self.site_specs[site]
            count = self.max_seqs
            for n in spec.shape:
                count *= int(n)
            total += count * torch.empty((), dtype=spec.dtype).element_size()
        return total

    def allocate_tensors(self, dtype: torch.dtype, device) -> None:
        """Per paged site: keys [num_blocks * pieces, kv_heads, kernel_block, head_dim] and
        values [num_blocks * pieces, kv_heads, head_dim, kernel_block] (transposed inside a
        page); state per state site: [max_seqs, *shape]."""
        for g in self.groups:
            pages = self.num_blocks * self.pieces
            k_shape = (pages, g.spec.num_kv_heads, self.kernel_block, g.spec.head_dim)
            v_shape = (pages, g.spec.num_kv_heads, g.spec.head_dim, self.kernel_block)
            for site in g.sites:
                self.kv[site] = (torch.zeros(k_shape, dtype=dtype, device=device),
                                 torch.zeros(v_shape, dtype=dtype, device=device))
        for site in self.state_sites:
            spec = self.site_specs[site]
            self.state[site] = torch.zeros((self.max_seqs,) + tuple(spec.shape), dtype=spec.dtype,
                                           device=device)

    # ------------------------------------------------------------------ requests
    def has(self, request: Hashable) -> bool:
        return request in self.requests

    def admit(self, request: Hashable) -> int:
        """Start a request: takes a state slot.  Raises OutOfPages if there is none."""
        if request in self.requests:
            raise ValueError(f"request {request!r} is already live")
        slot = self.slots.allocate()
        self.requests[request] = RequestState(slot)
        for g in self.groups:
            g.tables[request] = array("i")
        return slot

    def can_admit(self) -> bool:
        return self.slots.num_free() > 0

    def length(self, request: Hashable) -> int:
        return self.requests[request].length

    def slot(self, request: Hashable) -> int:
        return self.requests[request].slot

    def pages_needed(self, group: PageGroup, have_tokens: int, new_tokens: int) -> int:
        """Pages to take so that tokens [have, have + new) can be written."""
        return (_ceil_div(have_tokens + new_tokens, self.block_size)
                - _ceil_div(have_tokens, self.block_size))

    def can_reserve(self, request: Optional[Hashable], new_tokens: int,
                    already_taken: Optional[Dict[int, int]] = None) -> bool:
        """Whether every group has the pages for ``new_tokens`` more tokens of ``request``
        (None: a request that is not admitted yet).  ``already_taken[g]`` counts pages that
        the caller has promised to others in the same step."""
        st = self.requests.get(request) if request is not None else None
        have = (st.length + st.pending) if st else 0
        for gi, g in enumerate(self.groups):
            need = self.pages_needed(g, have, new_tokens)
            taken = already_taken.get(gi, 0) if already_taken else 0
            if need + taken > g.pool.num_free():
                return False
        return True

    def reserve(self, request: Hashable, new_tokens: int) -> None:
        """Take the pages for the next ``new_tokens`` tokens in every group, or none at all."""
        st = self.requests[request]
        if not self.can_reserve(request, new_tokens):
            raise OutOfPages(f"request {request!r}: no pages for {new_tokens} more tokens")
        have = st.length + st.pending
        for g in self.groups:
            need = self.pages_needed(g, have, new_tokens)
            g.tables[request].extend(g.pool.allocate_many(need))
        st.pending += new_tokens

    def cancel(self, request: Hashable) -> None:
        """The reserved tokens will not be written after all: the pages taken for them go
        back."""
        st = self.requests[request]
        keep = _ceil_div(st.length, self.block_size)
        for g in self.groups:
            table = g.tables[request]
            while len(table) > keep:
                page = table.pop()
                if page >= 0:
                    g.pool.free(page)
        st.pending = 0

    def commit(self, request: Hashable) -> None:
        """The reserved tokens have been written.  Pages that a window has passed go back."""
        st = self.requests[request]
        st.length += st.pending
        st.pending = 0
        st.started = True
        for g in self.groups:
            w = g.spec.window
            if w is None:
                continue
            # the next query is at position >= length and reads keys > position - w
            first_needed = st.length - w + 1
            table = g.tables[request]
            for idx in range(min(len(table), max(0, first_needed // self.block_size))):
                if table[idx] >= 0:
                    g.pool.free(table[idx])
                    table[idx] = -1

    def release(self, request: Hashable) -> None:
        """The request ends (or is preempted): everything it holds goes back."""
        st = self.requests.pop(request)
        for g in self.groups:
            for page in g.tables.pop(request):
                if page >= 0:
                    g.pool.free(page)
        self.slots.free(st.slot)

    # ------------------------------------------------------------------ views for a step
    def block_table(self, group_index: int, request: Hashable) -> List[int]:
        return list(self.groups[group_index].tables[request])

    def slot_of_token(self, group_index: int, request: Hashable, position: int) -> int:
        page = self.groups[group_index].tables[request][position // self.block_size]
        if page < 0:
            raise RuntimeError(f"request {request!r}: position {position} lies in a page that "
                               f"was given back")
        return page * self.block_size + position % self.block_size

    def num_free_blocks(self) -> int:
        return min((g.pool.num_free() for g in self.groups), default=self.num_blocks)

    def check(self) -> None:
        """Bookkeeping invariants: no page lost, held twice, or held by nobody."""
        for g in self.groups:
            g.pool.check()
            seen: List[int] = []
            for table in g.tables.values():
                seen.extend(p for p in table if p >= 0)
            if len(seen) != len(set(seen)):
                raise AssertionError("a page is in two block tables")
            if set(seen) != g.pool.held():
                raise AssertionError("held pages and block tables disagree")
        self.slots.check()
        if {s.slot for s in self.requests.values()} != self.slots._held:
            raise AssertionError("held slots and live requests disagree")
