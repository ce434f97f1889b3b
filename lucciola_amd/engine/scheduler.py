"""The continuous-batching scheduler: which requests run in the next step, and with how many
tokens each.  Host code only; it decides from the cache manager's bookkeeping.

What is kept from the reference (src/scheduler.cc:42-139): running requests are served first,
one decode token each; then prompts are cut into portions under what is left of the step's
token budget (576 there, src/scheduler.cc:48; 2,048 by default here), first come first served; the step that feeds a
prompt's last token makes its request running, and that step's logits give its first new
token (src/scheduler.cc:113-117).

What is different:
  * decode tokens count against the budget too (the reference bounds only the prompt portion,
    src/scheduler.cc:52-74 against :77);
  * several waiting requests may start in one step (the reference considers only the front
    one, src/scheduler.cc:77-78); the queue is never reordered: if the front request cannot
    go, none behind it does;
  * when a decode finds no free page the reference parks the request in ``swapped_`` for good
    (src/scheduler.cc:33-40, 57-64).  Here the most recently admitted request is preempted by
    recompute: all it holds goes back, it returns to the FRONT of the waiting queue, and its
    prompt and the tokens it has generated are fed again later; tokens already emitted are not
    emitted twice, and sampling goes on from the same draw index;
  * a request that could never fit (prompt + max_new_tokens beyond the pool or the model's
    positions) is refused when it is added.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional

from ..cache.manager import CacheManager
from .batch import StepEntry
from .sequence import Sequence, SequenceStatus


@dataclass
class ScheduledStep:
    entries: List[StepEntry] = field(default_factory=list)
    seqs: List[Sequence] = field(default_factory=list)
    samples: List[bool] = field(default_factory=list)   # does this entry yield a new token
    portions: List[int] = field(default_factory=list)   # prompt tokens fed by this entry (0: a decode)
    num_decode_seqs: int = 0
    num_prefill_seqs: int = 0
    num_prefill_tokens: int = 0
    preempted: List[Sequence] = field(default_factory=list)

    @property
    def num_seqs(self) -> int:
        return len(self.entries)

    @property
    def num_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)


class Scheduler:
    def __init__(self, cache: CacheManager, max_tokens_per_step: int = 2048,
                 max_seqs: Optional[int] = None, max_model_len: int = 0, portion_multiple: int = 1):
        self.cache = cache
        self.max_tokens_per_step = int(max_tokens_per_step)
        self.max_seqs = int(max_seqs or cache.max_seqs)
        self.max_model_len = int(max_model_len)
        # portions of a prompt, but for its last, are multiples of this (what the model's
        # mixers ask for, ``CausalLM.portion_multiple``)
        self.portion_multiple = max(1, int(portion_multiple))
        self.waiting: Deque[Sequence] = deque()
        self.running: List[Sequence] = []
        self.num_preemptions = 0

    # ------------------------------------------------------------------ requests
    def add_request(self, seq: Sequence) -> None:
        total = seq.get_prompt_len() + seq.params.max_new_tokens
        capacity = self.cache.num_blocks * self.cache.block_size
        if total > capacity:
            raise ValueError(f"request {seq.seq_id}: prompt {seq.get_prompt_len()} + "
                             f"max_new_tokens {seq.params.max_new_tokens} exceed the cache "
                             f"({capacity} tokens)")
        if self.max_model_len and total > self.max_model_len:
            raise ValueError(f"request {seq.seq_id}: prompt {seq.get_prompt_len()} + "
                             f"max_new_tokens {seq.params.max_new_tokens} exceed the model's "
                             f"{self.max_model_len} positions")
        seq.status = SequenceStatus.WAITING
        self.waiting.append(seq)

    def has_unfinished_requests(self) -> bool:
        return bool(self.waiting) or bool(self.running)

    def free_sequence(self, seq: Sequence) -> None:
        """The request is over: pages and slot go back (src/scheduler.cc:20-31)."""
        if self.cache.has(seq.seq_id):
            self.cache.release(seq.seq_id)
        seq.status = SequenceStatus.FINISHED
        if seq in self.running:
            self.running.remove(seq)
        elif seq in self.waiting:
            self.waiting.remove(seq)

    def _preempt(self, seq: Sequence) -> None:
        if self.cache.has(seq.seq_id):
            self.cache.release(seq.seq_id)
        seq.prefill_offset = 0
        seq.preemptions += 1
        seq.status = SequenceStatus.WAITING
        self.num_preemptions += 1
        if seq in self.running:
            self.running.remove(seq)
            self.waiting.appendleft(seq)
        # a partly fed waiting request stays where it is in the queue

    def _victim(self, keep: Sequence) -> Optional[Sequence]:
        """The most recently admitted request that holds something: a partly fed waiting
        request first, then the running ones from the back."""
        if self.waiting and self.waiting[0].prefill_offset > 0 and self.waiting[0] is not keep:
            return self.waiting[0]
        for seq in reversed(self.running):
            return seq
        return None

    # ------------------------------------------------------------------ one step
    def step(self) -> ScheduledStep:
        out = ScheduledStep()
        budget = self.max_tokens_per_step
        taken: Dict[int, int] = {}

        def note_pages(seq_id, have, n):
            for gi, g in enumerate(self.cache.groups):
                taken[gi] = taken.get(gi, 0) + self.cache.pages_needed(g, have, n)

        # 1. running requests: one token each
        for seq in list(self.running):
            if seq not in self.running:      # preempted while serving an earlier one
                continue
            if budget <= 0:
                break
            while not self.cache.can_reserve(seq.seq_id, 1, taken):
                victim = self._victim(keep=None)
                if victim is None:
                    break
                # entries already scheduled in this step keep their promise: never take a
                # request that is in `out`
                if victim in out.seqs:
                    victim = seq
                self._preempt(victim)
                out.preempted.append(victim)
                if victim is seq:
                    break
            if seq not in self.running:
                continue
            if not self.cache.can_reserve(seq.seq_id, 1, taken):
                continue
            note_pages(seq.seq_id, self.cache.length(seq.seq_id), 1)
            out.entries.append(StepEntry(seq.seq_id, [seq.token_ids[-1]], [0]))
            out.seqs.append(seq)
            out.samples.append(True)
            out.portions.append(0)
            out.num_decode_seqs += 1
            budget -= 1

        # 2. waiting requests, in order, portions under the remaining budget
        live = len(self.cache.requests)
        while self.waiting and budget > 0:
            seq = self.waiting[0]
            if seq in out.preempted:
                break   # preempted in this very step: it starts again in a later one
            known = self.cache.has(seq.seq_id)
            if not known and live >= self.max_seqs:
                break
            have = self.cache.length(seq.seq_id) if known else 0
            remaining = seq.get_len() - seq.prefill_offset
            chunk = min(budget, remaining)
            # shrink the portion to the pages that are free
            bs = self.cache.block_size
            fit = chunk
            for gi, g in enumerate(self.cache.groups):
                free = g.pool.num_free() - taken.get(gi, 0)
                room = (-have) % bs + max(free, 0) * bs
                fit = min(fit, room)
            chunk = fit
            if chunk < remaining:
                chunk -= chunk % self.portion_multiple
            if chunk <= 0:
                break
            if not known:
                live += 1
            note_pages(seq.seq_id, have, chunk)
            tokens = seq.token_ids[seq.prefill_offset:seq.prefill_offset + chunk]
            last = seq.prefill_offset + chunk >= seq.get_len()
            out.entries.append(StepEntry(seq.seq_id, tokens, [chunk - 1] if last else []))
            out.seqs.append(seq)
            out.samples.append(last)
            out.portions.append(chunk)
            out.num_prefill_seqs += 1
            out.num_prefill_tokens += chunk
            seq.prefill_offset += chunk
            budget -= chunk
            if last:
                self.waiting.popleft()
                seq.status = SequenceStatus.RUNNING
                self.running.append(seq)
            else:
                break   # the budget or the pages are used up
        return out

    def undo(self, step: ScheduledStep) -> None:
        """The step was not run: its prompt portions are waiting again, in their order.
        Requests that the step preempted stay preempted (they hold nothing, which is a state
        like any other)."""
        for seq, chunk, last in reversed(list(zip(step.seqs, step.portions, step.samples))):
            if chunk == 0:
                continue
            seq.prefill_offset -= chunk
            if last:
                self.running.remove(seq)
                self.waiting.appendleft(seq)
                seq.status = SequenceStatus.WAITING

    def on_token(self, seq: Sequence, token: int) -> bool:
        """Record a generated token; returns True if the request has finished."""
        seq.append_token_id(token)
        seq.prefill_offset = seq.get_len() - 1   # everything but the new token is cached
        return seq.should_stop()
