"""The cache manager: pages of keys and values with a block table per request, and slots for
per-request state of fixed size.

Every site of a model's run order states what it needs (:mod:`lucciola_amd.cache.specs`); a
need counts its own bytes and makes its own memory, the manager keeps the books.
Sites with equal paged needs form a *group*: one pool of page ids and one block table per
request serve the whole group, and each site of the group has key and value tensors of its
own that are indexed by those page ids.  Groups differ in what they keep: all keys, or a
window of them, in which case the pages the window has passed are given back after each step.

The reference has one group (every layer alike, src/qwen.cc:507-516), takes a page when
``ceil(len / block_size)`` exceeds the table (src/scheduler.cc:55-58,89-97) and gives all of
a request's pages back when it ends (src/scheduler.cc:20-31).  The bookkeeping here is host
code only; the device memory is made by the needs in :meth:`CacheManager.allocate_tensors`.
"""
from __future__ import annotations

from array import array
from dataclasses import dataclass, field
from typing import Any, Dict, Hashable, List, Optional, Sequence, Tuple

import torch

from .page_pool import OutOfPages, PagePool, SlotPool
from .specs import CacheLayout, CacheNeed


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


@dataclass
class PageGroup:
    spec: CacheNeed
    sites: List[int]
    pool: PagePool
    kernel_page: int          # tokens of a page as the group's kernels index it
    pieces: int               # kernel pages in one of the manager's pages
    # a request's page ids in order, as a typed array (numpy views it without a copy); -1: given back
    tables: Dict[Hashable, array] = field(default_factory=dict)


@dataclass
class RequestState:
    slot: int
    length: int = 0           # tokens whose keys/values (or state) are in the cache
    pending: int = 0          # tokens reserved by `reserve` and not yet committed
    started: bool = False     # False until the first commit: state slots are zeroed then


class CacheManager:
    def __init__(self, site_specs: Sequence[Optional[object]], block_size: int, num_blocks: int,
                 max_seqs: int, scatter_pages: bool = True):
        """``site_specs[i]``: what site i of the run order needs: a :class:`CacheNeed`, a
        tuple of them (a layer with several caching parts, in the order of its slots) or
        None.  A site that reads another site's cache is passed as None here.
        ``scatter_pages``: see :class:`PagePool`."""
        if block_size <= 0 or num_blocks <= 0:
            raise ValueError("block_size and num_blocks must be positive")
        self.block_size = block_size
        self.num_blocks = num_blocks
        self.max_seqs = max_seqs
        self.site_needs: List[Tuple[CacheNeed, ...]] = []
        for i, spec in enumerate(site_specs):
            needs = () if spec is None else tuple(spec) if isinstance(spec, (tuple, list)) else (spec,)
            for need in needs:
                if not isinstance(need, CacheNeed):
                    raise TypeError(f"site {i}: {need!r} is not a cache need")
            self.site_needs.append(needs)
        # What a group's kernels see: where a need's kernels are built for a smaller page than
        # the manager's (a page of 32, 48, 64, ... tokens for kernels made for 16), a page lies
        # in memory as that many kernel pages in a row, and the block tables that go to the
        # device name those (page p becomes p * pieces ... p * pieces + pieces - 1).  A slot id,
        # page * block_size + offset, is the same number either way.
        self.groups: List[PageGroup] = []
        self.need_group: Dict[Tuple[int, int], int] = {}     # (site, which of its needs) -> group
        for i, needs in enumerate(self.site_needs):
            for k, need in enumerate(needs):
                if not need.paged:
                    continue
                for gi, g in enumerate(self.groups):
                    if g.spec == need:
                        g.sites.append(i)
                        self.need_group[(i, k)] = gi
                        break
                else:
                    page = int(need.kernel_page(block_size))
                    if page <= 0 or block_size % page:
                        raise ValueError(f"site {i}: a kernel page of {page} tokens does not divide "
                                         f"the page size {block_size}")
                    self.groups.append(PageGroup(need, [i], PagePool(num_blocks, scatter_pages),
                                                 page, block_size // page))
                    self.need_group[(i, k)] = len(self.groups) - 1
        self.has_fixed_state = any(not need.paged for needs in self.site_needs for need in needs)
        self.slots = SlotPool(max_seqs)
        self.requests: Dict[Hashable, RequestState] = {}
        # device memory (made by allocate_tensors): per site, what each of its needs allocated
        self.storage: Dict[int, Tuple[Any, ...]] = {}

    # ------------------------------------------------------------------ tensors
    def bytes_per_block(self, dtype: torch.dtype) -> int:
        """Bytes that one page costs over all paged sites."""
        return sum(len(g.sites) * g.spec.bytes_per_page(self.block_size, dtype) for g in self.groups)

    def state_bytes(self, dtype: torch.dtype = torch.float32) -> int:
        """Bytes of the per-request pieces of all fixed needs."""
        return sum(self.max_seqs * need.bytes_per_request(dtype)
                   for needs in self.site_needs for need in needs if not need.paged)

    def layout_of(self, site: int, which: int) -> CacheLayout:
        gi = self.need_group.get((site, which))
        page = self.groups[gi].kernel_page if gi is not None else self.block_size
        return CacheLayout(self.num_blocks, self.block_size, page, self.max_seqs)

    def allocate_tensors(self, dtype: torch.dtype, device) -> None:
        """Every need makes its own memory (``CacheNeed.allocate``); the manager keeps it by site
        and hands it to the site's view of a step."""
        for i, needs in enumerate(self.site_needs):
            if needs:
                self.storage[i] = tuple(need.allocate(self.layout_of(i, k), dtype, device)
                                        for k, need in enumerate(needs))

    def start_slots(self, slots: Sequence[int]) -> None:
        """Requests begin in these slots: every need brings its memory there to its initial state."""
        for i, stored in self.storage.items():
            for need, storage in zip(self.site_needs[i], stored):
                for slot in slots:
                    need.start(storage, slot)

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
