"""The step function: one batch of (request, its next tokens) through the model, from the cache.

``ModelRunner.step`` runs only the tokens it is given, as one batch, and returns float32
logits at the wanted places.  It is what the scheduler, the entry points and the trace replay
all call; nothing else runs the model.  The reference's counterpart is
``QwenModel::step_with_paged_attention`` (src/qwen.cc:801-902), which also picks the next
token and appends it to the sequences itself; here sampling is a stage of its own.
"""
from __future__ import annotations

import time
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.page_pool import OutOfPages
from ..config.engine_config import EngineConfig
from ..models.causal_lm import CausalLM
from ..kernels import ops
from .batch import PENDING, Carry, SiteView, StepBatch, StepEntry, build_batch, prepare_batch, upload_batch


class _CapturedStep:
    def __init__(self, graph, batch, sites, logits):
        self.graph, self.batch, self.sites, self.logits = graph, batch, sites, logits


def blocks_from_free_memory(free: int, bytes_per_block: int, state_bytes: int,
                            config: EngineConfig, max_positions: int = 0) -> int:
    """Pages for the cache when none are asked for, as the reference sizes its pools
    (src/qwen.cc:527-543): ``memory_fraction`` of the free memory less a reserve, divided by
    what a page costs over all layers.  Beyond the reference: the per-request state tensors
    come off first, and the count is capped at what ``max_seqs`` requests of the model's
    longest context can hold and at what a 32-bit slot id (page * block_size + offset) can
    name."""
    per_block = max(1, int(bytes_per_block))
    usable = int(max(0, free - config.memory_reserve) * config.memory_fraction) - int(state_bytes)
    blocks = usable // per_block
    if blocks <= 0:
        raise RuntimeError(f"no memory for the cache: {free} bytes free, a page of all "
                           f"layers takes {per_block}")
    blocks = min(blocks, (2 ** 31 - 1) // config.block_size)
    if max_positions:
        blocks = min(blocks, config.max_seqs * -(-max_positions // config.block_size))
    return int(blocks)


class ModelRunner:
    def __init__(self, model: CausalLM, config: EngineConfig, num_blocks: Optional[int] = None):
        self.model = model
        self.config = config
        self.device = model.ctx.device
        needs = model.site_needs()
        blocks = num_blocks if num_blocks is not None else config.max_blocks
        if blocks <= 0:
            blocks = self._blocks_from_free_memory(needs)
        self.cache = CacheManager(needs, config.block_size, blocks, config.max_seqs)
        self.cache.allocate_tensors(config.dtype, self.device)
        self.planners = model.batch_planners()
        self.steps = 0
        self.tokens = 0
        # seconds of host time spent in `step`, by what it went to: checking the entries and
        # reserving pages, laying out the batch and sending it, queueing the model's kernels
        # (or replaying the captured step)
        self.times = {"reserve": 0.0, "batch": 0.0, "launch": 0.0}
        # decode steps replayed from HIP graphs: (requests, block-table width) -> captured step
        self.use_graphs = (config.use_graphs and self.device.type == "cuda"
                           and config.dtype == torch.bfloat16 and model.graph_safe())
        self._graphs: Dict[tuple, "_CapturedStep"] = {}
        self._graph_epoch = None
        self.graph_replays = 0
        self.graph_captures = 0

    # ------------------------------------------------------------------ sizing
    def _blocks_from_free_memory(self, needs) -> int:
        probe = CacheManager(needs, self.config.block_size, 1, self.config.max_seqs)
        free, _ = torch.cuda.mem_get_info(self.device)
        return blocks_from_free_memory(
            free, probe.bytes_per_block(self.config.dtype), probe.state_bytes(self.config.dtype), self.config,
            self.model.spec.max_positions)

    # ------------------------------------------------------------------ the step
    def can_run(self, entries: Sequence[StepEntry]) -> bool:
        taken: Dict[int, int] = {}
        new_requests = 0
        for e in entries:
            known = self.cache.has(e.request)
            if not known:
                new_requests += 1
            if not self.cache.can_reserve(e.request if known else None, len(e.tokens), taken):
                return False
            have = (self.cache.length(e.request)) if known else 0
            for gi, g in enumerate(self.cache.groups):
                taken[gi] = taken.get(gi, 0) + self.cache.pages_needed(g, have, len(e.tokens))
        return new_requests <= self.cache.slots.num_free()

    def step(self, entries: Sequence[StepEntry], carry: Optional[Carry] = None) -> torch.Tensor:
        """Run the entries as one batch; returns float32 logits [wanted places, vocab] in the
        order of the entries and of each entry's ``want``.

        Nothing here waits for the GPU: the kernels are queued on the current stream and the
        logits are read in stream order.  An entry whose only token is ``PENDING`` takes the id
        that ``carry`` holds for its request, on the device: a caller may queue a request's
        next step before it has seen the token that the last one sampled.

        A request that the cache does not know is admitted.  Raises OutOfPages if the pages or
        slots for the whole batch are not there.  Whatever is raised, by the checks or by the
        model, the cache's bookkeeping is left as it was before the call."""
        entries = [e for e in entries if len(e.tokens) > 0]
        V = self.model.vocab_size
        if not entries:
            return torch.empty((0, V), dtype=torch.float32, device=self.device)
        names = [e.request for e in entries]
        if len(set(names)) != len(names):
            twice = next(n for n in names if names.count(n) > 1)
            raise ValueError(f"request {twice!r} appears twice in one step")
        limit = self.model.spec.max_positions
        fed = [e for e in entries if len(e.tokens) == 1 and e.tokens[0] == PENDING]
        if fed:
            if carry is None:
                raise ValueError(f"request {fed[0].request!r}: a pending token and no carry to take it from")
            for e in fed:
                if not 0 <= carry.rows.get(e.request, -1) < carry.ids.shape[0]:
                    raise ValueError(f"request {e.request!r}: no row in the step's carry")
        known = [e for e in entries if not (len(e.tokens) == 1 and e.tokens[0] == PENDING)] if fed else entries
        if all(len(e.tokens) == 1 for e in known):      # one check for a step of single tokens
            if known:
                self._check_ids(np.asarray([e.tokens[0] for e in known]), known)
        else:
            for e in known:
                self._check_ids(np.asarray(e.tokens), [e])
        if limit:
            for e in entries:
                have = self.cache.length(e.request) if self.cache.has(e.request) else 0
                if have + len(e.tokens) > limit:
                    raise ValueError(f"request {e.request!r}: {have + len(e.tokens)} tokens exceed "
                                     f"the model's {limit} positions")
        if not self.can_run(entries):
            raise OutOfPages(f"the cache cannot take this step ({sum(len(e.tokens) for e in entries)}"
                             f" tokens of {len(entries)} requests; "
                             f"{self.cache.num_free_blocks()} pages free)")
        fresh: List[int] = []
        admitted: List[Hashable] = []
        clock = time.perf_counter
        t_in = clock()
        try:
            for e in entries:
                if not self.cache.has(e.request):
                    self.cache.admit(e.request)
                    admitted.append(e.request)
                if self.cache.length(e.request) == 0:
                    fresh.append(self.cache.slot(e.request))
                self.cache.reserve(e.request, len(e.tokens))
            if fresh:
                self.cache.start_slots(fresh)
            t_reserved = clock()
            self.times["reserve"] += t_reserved - t_in

            if self.use_graphs and len(entries) <= self.config.graph_max_batch and all(
                    len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
                logits, num_tokens = self._graph_step(entries, carry if fed else None), len(entries)
            else:
                batch = build_batch(entries, self.cache, self.device,
                                    carry_rows=carry.rows if fed else None, planners=self.planners)
                t_built = clock()
                self.times["batch"] += t_built - t_reserved
                if fed:
                    ops.feed_tokens(batch.token_ids, batch.feed, carry.ids)
                logits, num_tokens = self.model.forward(batch, self._sites(batch)), batch.num_tokens
                self.times["launch"] += clock() - t_built
        except BaseException:
            # nothing of this step counts: reserved pages go back, requests that it admitted
            # leave again (what kernels may already have written lies beyond every length)
            for e in entries:
                if self.cache.has(e.request):
                    if e.request in admitted:
                        self.cache.release(e.request)
                    else:
                        self.cache.cancel(e.request)
            raise
        for e in entries:
            self.cache.commit(e.request)
        self.steps += 1
        self.tokens += num_tokens
        return logits

    def _check_ids(self, ids: np.ndarray, entries: Sequence[StepEntry]) -> None:
        V = self.model.vocab_size
        who = entries[0].request if len(entries) == 1 else [e.request for e in entries]
        if ids.dtype.kind not in "iu":
            raise ValueError(f"request {who!r}: token ids must be integers")
        if int(ids.min()) < 0 or int(ids.max()) >= V:
            bad = int(ids[(ids < 0) | (ids >= V)][0])
            raise ValueError(f"request {who!r}: token id {bad} is outside the vocabulary of {V}")

    # ------------------------------------------------------------------ graph replay
    def _graph_step(self, entries: Sequence[StepEntry], carry: Optional[Carry]) -> torch.Tensor:
        """A step of single tokens, one per request, each wanting its logits: captured once per
        (number of requests, block-table width, what the planners say of the launches' shapes) as
        a HIP graph and replayed afterwards.  Only the batch description changes between replays,
        and it lives in one device buffer that is overwritten in place.  """
        widest = max((len(g.tables[e.request]) for g in self.cache.groups for e in entries),
                     default=1)
        pad = max(64, -(-widest // 64) * 64)
        # batches of 5 or more requests are filled up to a multiple of 8 with copies of the
        # first entry (same token, same position, same cache slot: the copies compute and write
        # what the original does), so that a batch that shrinks by one does not need a new graph;
        # not with per-request state, which a copy would update a second time
        real = len(entries)
        rows = real if real <= 4 or self.cache.has_fixed_state else -(-real // 8) * 8
        entries = list(entries) + [entries[0]] * (rows - real)
        epoch = self.model.tables_epoch()
        if epoch != self._graph_epoch:      # a part has made a table anew: addresses changed
            self._graphs.clear()
            self._graph_epoch = epoch
        t_in = time.perf_counter()
        prepared = prepare_batch(entries, self.cache, pad_blocks=pad,
                                 carry_rows=carry.rows if carry else None, planners=self.planners)
        # a kernel's launch may depend on more than the layout (the attention's shares on how
        # uneven the requests' lengths are): a captured step serves the batches of its own kind
        key = (rows, pad, prepared.graph_hint)
        captured = self._graphs.get(key)
        next_position = max(self.cache.length(e.request) for e in entries)
        if captured is None or not self.model.ready(next_position):
            batch = upload_batch(prepared, self.device)
            if carry:
                ops.feed_tokens(batch.token_ids, batch.feed, carry.ids)
            sites = self._sites(batch)
            logits = self.model.forward(batch, sites)       # runs the step (and grows tables)
            if self.model.tables_epoch() != epoch:
                self._graphs.clear()
                self._graph_epoch = self.model.tables_epoch()
            if len(self._graphs) >= self.config.graph_cache_size:
                self._graphs.pop(next(iter(self._graphs)))
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_logits = self.model.forward(batch, sites)
            self._graphs[key] = _CapturedStep(graph, batch, sites, static_logits)
            self.graph_captures += 1
            self.times["launch"] += time.perf_counter() - t_in      # a capture: the step run twice
            return logits[:real]
        upload_batch(prepared, self.device, into=captured.batch.buffer, refresh_only=True)
        t_built = time.perf_counter()
        if carry:       # outside the graph: the carry is at another address every step
            ops.feed_tokens(captured.batch.token_ids, captured.batch.feed, carry.ids)
        captured.graph.replay()
        self.graph_replays += 1
        logits = captured.logits[:real].clone()      # the next replay overwrites the graph's own output
        self.times["batch"] += t_built - t_in
        self.times["launch"] += time.perf_counter() - t_built
        return logits

    def _sites(self, batch: StepBatch) -> List[SiteView]:
        sites = []
        cache = self.cache
        for index, entry in enumerate(self.model.spec.run_order):
            owner = index if entry.cache_of is None else entry.cache_of
            stored = cache.storage.get(owner, ())
            views = tuple(batch.groups[cache.need_group[(owner, k)]] if (owner, k) in cache.need_group else None
                          for k in range(len(stored)))
            sites.append(SiteView(batch=batch, index=index, writes_cache=entry.cache_of is None,
                                  caches=stored, page_views=views))
        return sites

    def finish(self, request: Hashable) -> None:
        """The request is over: its pages and its slot go back."""
        if self.cache.has(request):
            self.cache.release(request)
