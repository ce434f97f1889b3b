"""A request as the scheduler sees it (reference: include/sequence.h:10-42)."""
from __future__ import annotations

import enum
from typing import List, Optional, Sequence as Seq

from ..sampling.sampler import SamplingParams


class SequenceStatus(enum.Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


class Sequence:
    """Token ids of a request (prompt, then generated), and how far its prompt has been fed.

    ``prefill_offset`` counts the tokens whose keys and values are cached; after a
    preemption it goes back to 0 and everything known so far, generated tokens included,
    is fed again as a prompt."""

    def __init__(self, seq_id: int, prompt_token_ids: Seq[int],
                 params: Optional[SamplingParams] = None):
        if len(prompt_token_ids) == 0:
            raise ValueError("a request needs at least one prompt token")
        self.seq_id = seq_id
        self.status = SequenceStatus.WAITING
        self.prompt_len = len(prompt_token_ids)
        self.token_ids: List[int] = [int(t) for t in prompt_token_ids]
        self.prefill_offset = 0
        self.params = params or SamplingParams()
        self.preemptions = 0

    def get_seq_id(self) -> int:
        return self.seq_id

    def get_len(self) -> int:
        return len(self.token_ids)

    def get_prompt_len(self) -> int:
        return self.prompt_len

    def get_token_ids(self) -> List[int]:
        return self.token_ids

    @property
    def num_generated(self) -> int:
        return len(self.token_ids) - self.prompt_len

    @property
    def output_token_ids(self) -> List[int]:
        return self.token_ids[self.prompt_len:]

    def append_token_id(self, token_id: int) -> None:
        self.token_ids.append(int(token_id))

    def is_finished(self) -> bool:
        return self.status is SequenceStatus.FINISHED

    def should_stop(self) -> bool:
        """Stop rules of the reference's engine loop (src/async_engine.cc:143-147): an
        end-of-sequence id, or max_new_tokens generated."""
        if self.num_generated >= self.params.max_new_tokens:
            return True
        return bool(self.num_generated) and self.stops_on(self.token_ids[-1])

    def stops_on(self, token: int) -> bool:
        """Is this generated token an end-of-sequence id that the request heeds."""
        return not self.params.ignore_eos and token in self.params.eos_token_ids
