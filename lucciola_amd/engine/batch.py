"""The description of one step's batch, as the model and its kernels see it.

The reference's ``InputMetadata`` (include/sequence.h:46-61) holds decode tokens first and
then at most one prompt portion; here a batch is any list of (request, next tokens) entries:
portions of prompts beside single decoded tokens, in any order and of any length >= 1.
Everything the kernels index by is built on the host from the cache manager's tables and
sent to the GPU in one copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager

PENDING = -1        # a token that an earlier step has sampled and the host has not seen yet


@dataclass
class HostLayout:
    """A step's batch as the host knows it, for the parts' planners (``Part.batch_planner``)."""

    num_requests: int
    num_tokens: int
    q_start: List[int]          # token offset of each request in the batch, R + 1 entries
    first_position: List[int]   # cached length of each request before this step
    block_size: int
    single: bool                # every request brings one token and wants its logits


@dataclass
class Plan:
    """What a planner made of a step's batch: its arrays on the device, its numbers."""

    arrays: Dict[str, torch.Tensor]
    info: Dict[str, Any]
    made: Dict[Any, Any] = field(default_factory=dict)   # for the parts: what they derive from it


@dataclass
class StepEntry:
    """A request's next tokens, and the places among them whose logits are wanted."""

    request: Hashable
    tokens: Sequence[int]       # [PENDING]: the token comes from the carry given to the step
    want: Sequence[int] = ()


@dataclass
class Carry:
    """Tokens that an earlier step sampled, still on the device: ``ids[rows[request]]`` is the
    next token of ``request``."""

    ids: torch.Tensor           # int32 [S]
    rows: dict


@dataclass
class PagesView:
    """What a step looks like to one group of cache pages: the pages every request of the batch
    holds and the place where each token's own entry is written.  All tensors are int32 on the
    device.  Parts that keep paged memory read it through this; what a part's kernels want
    beyond it (work lists, records of their own) the part derives itself and may keep in
    ``made``, which lives as long as the batch (through every replay of a captured step)."""

    block_table: torch.Tensor   # [R, width] page of position // page_size, in kernel pages; -1: given back
    slots: torch.Tensor         # [T] page * page_size + offset of each token of the batch; -1: none
    page_size: int              # tokens of a page as the group's kernels index it
    made: Dict[Any, Any] = field(default_factory=dict)


@dataclass
class SiteView:
    """What one site of the run order sees of the step: the batch and its own cache.

    ``caches[k]`` is what the k-th need of the site's layer allocated (``CacheNeed.allocate``:
    a tensor, a tuple of tensors, ...), ``page_views[k]`` the view of that need's page group
    (None for a need without pages).  A layer with one caching part, the usual case, reads
    ``site.cache`` and ``site.pages``; an arrangement with several hands ``site.part(k)`` to
    the k-th of them."""

    batch: "StepBatch"
    index: int
    writes_cache: bool
    caches: Tuple[Any, ...] = ()
    page_views: Tuple[Optional[PagesView], ...] = ()

    @property
    def cache(self) -> Any:
        return self.caches[0] if self.caches else None

    @property
    def pages(self) -> Optional[PagesView]:
        return self.page_views[0] if self.page_views else None

    def part(self, k: int) -> "SiteView":
        return SiteView(self.batch, self.index, self.writes_cache, self.caches[k:k + 1],
                        self.page_views[k:k + 1])


@dataclass
class StepBatch:
    num_tokens: int
    num_requests: int
    requests: List[Hashable]
    q_start: List[int]            # host: token offset of each request in the batch, R + 1 entries
    first_position: List[int]     # host: cached length of each request before this step
    slot_list: List[int]          # host: state slot of each request
    max_position: int
    token_ids: torch.Tensor       # int32 [T]
    positions: torch.Tensor       # int32 [T]
    tok_req: torch.Tensor         # int32 [T]
    want_rows: torch.Tensor       # int32 [W] rows of the batch whose logits are wanted
    slot_ids: torch.Tensor        # int32 [R]
    feed: torch.Tensor            # int32 [T] row of the carry a token is taken from, or -1
    q_offsets: Optional[torch.Tensor] = None   # int32 [R + 1]: q_start on the device
    ctx_len: Optional[torch.Tensor] = None     # int32 [R]: cached length of each request after this step
    max_ctx: int = 0              # the longest of them (of a captured step: what its layout allows)
    groups: List[PagesView] = field(default_factory=list)   # by page group of the cache manager
    plans: Dict[Any, Plan] = field(default_factory=dict)   # by planner key
    num_wanted: int = 0
    buffer: Optional[torch.Tensor] = None   # the one device buffer all of the above view


class _Packer:
    """Collects int32 arrays, sends them in one copy, and hands out views of the device copy."""

    def __init__(self) -> None:
        self._arrays: List[np.ndarray] = []
        self._offsets: List[int] = []
        self._size = 0

    def add(self, values, shape=None) -> int:
        arr = np.asarray(values, dtype=np.int32).reshape(-1)
        self._arrays.append(arr)
        self._offsets.append(self._size)
        self._size += int(arr.size)
        self._size = (self._size + 3) & ~3   # keep every array 16-byte aligned
        return len(self._arrays) - 1

    def upload(self, device, into: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Send everything in one copy; ``into``: a device buffer of an earlier batch with the
        very same layout, which is overwritten (so that kernels captured in a graph see the
        new values at the old addresses)."""
        host = np.zeros(max(self._size, 4), dtype=np.int32)
        for arr, off in zip(self._arrays, self._offsets):
            host[off:off + arr.size] = arr
        dev = torch.device(device)
        if into is not None and into.numel() != host.size:
            raise ValueError("the batch does not have the layout of the buffer it is to reuse")
        if dev.type == "cuda":
            staging = torch.empty(host.size, dtype=torch.int32, pin_memory=True)
            staging.numpy()[:] = host
            if into is not None:
                into.copy_(staging, non_blocking=True)
                self._dev = into
            else:
                self._dev = staging.to(dev, non_blocking=True)
        elif into is not None:
            into.copy_(torch.from_numpy(host))
            self._dev = into
        else:
            self._dev = torch.from_numpy(host).to(dev)
        return self._dev

    def view(self, handle: int, shape=None) -> torch.Tensor:
        off, n = self._offsets[handle], self._arrays[handle].size
        t = self._dev[off:off + n]
        return t.view(shape) if shape is not None else t


@dataclass
class PreparedBatch:
    """A step's batch laid out on the host, before anything is sent: what ``upload_batch`` needs,
    and ``graph_hint``, what the planners say about the shape of the kernels' launches for this
    batch beyond its layout (a captured step is replayed only for batches of the same hint)."""

    packer: "_Packer"
    handles: Dict[str, int]
    group_handles: list
    planned: list
    num_requests: int
    num_tokens: int
    requests: List[Hashable]
    q_start: List[int]
    first_position: List[int]
    slot_list: List[int]
    max_position: int
    max_ctx: int
    num_wanted: int
    graph_hint: tuple


def build_batch(entries: Sequence[StepEntry], cache: CacheManager, device,
                pad_blocks: Optional[int] = None, into: Optional[torch.Tensor] = None,
                refresh_only: bool = False, carry_rows: Optional[dict] = None,
                planners: Optional[Dict[Any, Callable]] = None) -> Optional[StepBatch]:
    """Lay the entries out as one flat batch.  Pages for the new tokens must be reserved.

    ``pad_blocks``: width of the block tables (at least the longest table), so that batches of
    the same make-up have the same layout; ``into``: the buffer of such an earlier batch;
    ``refresh_only``: only bring that buffer up to date (its views exist already), return None;
    ``carry_rows``: for entries whose one token is PENDING, the row of the carry it comes from
    (the caller copies it in on the device; the host's copy holds token 0 there);
    ``planners``: the model's ``batch_planners()``, whose arrays travel in the same copy."""
    prepared = prepare_batch(entries, cache, pad_blocks, carry_rows, planners)
    return upload_batch(prepared, device, into, refresh_only)


def prepare_batch(entries: Sequence[StepEntry], cache: CacheManager, pad_blocks: Optional[int] = None,
                  carry_rows: Optional[dict] = None,
                  planners: Optional[Dict[Any, Callable]] = None) -> PreparedBatch:
    """The host's half of ``build_batch``: every array of the batch and of the planners, packed
    for one copy, nothing sent yet."""
    bs = cache.block_size
    R = len(entries)
    requests = [e.request for e in entries]
    first_pos = [cache.length(req) for req in requests]
    slot_list = [cache.slot(req) for req in requests]
    single = all(len(e.tokens) == 1 and len(e.want) == 1 and int(e.want[0]) == 0 for e in entries)
    if single:
        # a step of single tokens, each wanting its logits: everything is one array operation
        T = R
        q_start = list(range(R + 1))
        token_ids = np.fromiter((e.tokens[0] for e in entries), dtype=np.int32, count=R)
        positions = np.asarray(first_pos, dtype=np.int32)
        tok_req = np.arange(R, dtype=np.int32)
        want_rows = tok_req
        ctx_len = positions + 1
    else:
        q_start = [0]
        token_parts, position_parts, req_parts = [], [], []
        want_rows = []
        for r, e in enumerate(entries):
            n = len(e.tokens)
            base = first_pos[r]
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise ValueError(f"request {e.request!r}: wanted place {w} is outside its {n} tokens")
                want_rows.append(q_start[-1] + int(w))
            token_parts.append(np.asarray(e.tokens, dtype=np.int32))
            position_parts.append(np.arange(base, base + n, dtype=np.int32))
            req_parts.append(np.full(n, r, dtype=np.int32))
            q_start.append(q_start[-1] + n)
        T = q_start[-1]
        token_ids = np.concatenate(token_parts) if token_parts else np.zeros(0, np.int32)
        positions = np.concatenate(position_parts) if position_parts else np.zeros(0, np.int32)
        tok_req = np.concatenate(req_parts) if req_parts else np.zeros(0, np.int32)
        ctx_len = [first_pos[r] + (q_start[r + 1] - q_start[r]) for r in range(R)]

    feed = np.full(T, -1, dtype=np.int32)
    pending = np.nonzero(token_ids == PENDING)[0]
    if pending.size:
        starts = {q_start[r]: r for r in range(R) if q_start[r + 1] - q_start[r] == 1}
        for i in pending.tolist():
            r = starts.get(i)
            if r is None or carry_rows is None or requests[r] not in carry_rows:
                raise ValueError(f"request {requests[int(tok_req[i])]!r}: a pending token must be "
                                 "an entry's only token and have a row in the step's carry")
            feed[i] = carry_rows[requests[r]]
        token_ids = token_ids.copy()
        token_ids[pending] = 0

    pk = _Packer()
    h_tok = pk.add(token_ids)
    h_feed = pk.add(feed)
    h_pos = pk.add(positions)
    h_req = pk.add(tok_req)
    h_want = pk.add(want_rows)
    h_slot = pk.add(slot_list)
    h_qs = pk.add(q_start)
    h_ctx = pk.add(ctx_len)
    num_wanted = len(want_rows)
    layout = HostLayout(R, T, q_start, first_pos, bs, single)
    planned = []
    for key, plan in (planners or {}).items():
        arrays, info = plan(layout)
        planned.append((key, {name: (pk.add(a), tuple(np.shape(a))) for name, a in arrays.items()}, info))

    group_handles = []
    for gi, g in enumerate(cache.groups):
        tables = [g.tables[req] for req in requests]
        mb = max((len(t) for t in tables), default=1) or 1
        if pad_blocks is not None:
            if pad_blocks < mb:
                raise ValueError(f"pad_blocks {pad_blocks} is below the longest block table {mb}")
            mb = pad_blocks
        flat = np.full((R, mb), -1, dtype=np.int32)
        for r, t in enumerate(tables):
            if len(t):
                flat[r, :len(t)] = np.frombuffer(t, dtype=np.int32)
        pages = flat[tok_req, positions // bs] if T else np.zeros(0, np.int32)
        slots = np.where(pages >= 0, pages * bs + positions % bs, -1).astype(np.int32)
        if g.pieces > 1:        # the kernels' pages: every page as its pieces in a row
            pieces = g.pieces
            flat = np.where(flat[:, :, None] >= 0,
                            flat[:, :, None] * pieces + np.arange(pieces, dtype=np.int32), -1)
            flat = flat.reshape(R, mb * pieces).astype(np.int32)
            mb *= pieces
        group_handles.append((pk.add(flat), mb, pk.add(slots), g.kernel_page))

    max_ctx = int(max(ctx_len)) if R else 0
    if pad_blocks is not None:
        max_ctx = pad_blocks * bs      # what the layout allows, not what this batch holds
    hint = tuple(info.get("graph_hint") for _, _, info in planned)
    return PreparedBatch(
        packer=pk, handles={"tok": h_tok, "feed": h_feed, "pos": h_pos, "req": h_req, "want": h_want,
                            "slot": h_slot, "qs": h_qs, "ctx": h_ctx},
        group_handles=group_handles, planned=planned, num_requests=R, num_tokens=T, requests=requests,
        q_start=q_start, first_position=first_pos, slot_list=slot_list,
        max_position=int(positions.max()) if T else 0, max_ctx=max_ctx, num_wanted=num_wanted,
        graph_hint=hint)


def upload_batch(prepared: PreparedBatch, device, into: Optional[torch.Tensor] = None,
                 refresh_only: bool = False) -> Optional[StepBatch]:
    """The other half: one copy to the device (``into``: over the buffer of an earlier batch of
    the same layout) and, unless ``refresh_only``, the views of it."""
    pk, h, R = prepared.packer, prepared.handles, prepared.num_requests
    buffer = pk.upload(device, into)
    if refresh_only:
        return None
    groups = [PagesView(block_table=pk.view(h_bt, (R, mb)), slots=pk.view(h_sl), page_size=page)
              for (h_bt, mb, h_sl, page) in prepared.group_handles]
    plans = {key: Plan({name: pk.view(hd, shape) for name, (hd, shape) in handles.items()}, info)
             for key, handles, info in prepared.planned}
    return StepBatch(
        num_tokens=prepared.num_tokens, num_requests=R, requests=prepared.requests, q_start=prepared.q_start,
        first_position=prepared.first_position, slot_list=prepared.slot_list,
        max_position=prepared.max_position,
        token_ids=pk.view(h["tok"]), positions=pk.view(h["pos"]), tok_req=pk.view(h["req"]),
        want_rows=pk.view(h["want"]), slot_ids=pk.view(h["slot"]), feed=pk.view(h["feed"]),
        q_offsets=pk.view(h["qs"]), ctx_len=pk.view(h["ctx"]), max_ctx=prepared.max_ctx, groups=groups,
        plans=plans, num_wanted=prepared.num_wanted, buffer=buffer)
