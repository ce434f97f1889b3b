"""Sampling the next token from the step's logits.

The reference picks the argmax on the device (src/kernels/argmax.cu) and has no other way of
sampling (temperature is future work there, docs/qwen_operators_guide.md:60).  Here a request
carries :class:`SamplingParams`; temperature 0 is greedy, otherwise the token is drawn from
softmax(logits / temperature) by inverse CDF with a uniform number that depends only on the
request's seed and on how many tokens it has generated: the draw is the same whatever else
is in the batch and survives preemption.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence, Tuple

import numpy as np
import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


def _mix(x: int) -> int:
    """splitmix64 finaliser."""
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform_for(seed: int, index: int) -> float:
    """A number in [0, 1) from (seed, index of the generated token), 24 bits wide so that it
    is exact in float32."""
    return (_mix(_mix(seed & _MASK) ^ (index & _MASK)) >> 40) / float(1 << 24)


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0
    seed: int = 0
    eos_token_ids: Tuple[int, ...] = ()
    ignore_eos: bool = False

    def __post_init__(self) -> None:
        if self.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        self.eos_token_ids = tuple(int(t) for t in self.eos_token_ids)


class SampledTokens:
    """The tokens one step sampled: ``ids`` (int32, on the logits' device) exists as soon as the
    kernels are queued, and may feed the next step from there; ``tokens()`` waits for the copy
    to the host."""

    def __init__(self, ids: torch.Tensor):
        self.ids = ids
        self._list = None
        self._event = None
        if ids.device.type == "cuda":
            self._host = torch.empty(ids.shape, dtype=ids.dtype, pin_memory=True)
            self._host.copy_(ids, non_blocking=True)
            self._event = torch.cuda.Event()
            self._event.record()
        else:
            self._host = ids

    def tokens(self) -> List[int]:
        if self._list is None:
            if self._event is not None:
                self._event.synchronize()
            self._list = [int(t) for t in self._host.tolist()]
        return self._list


class Sampler:
    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams],
               generated: Sequence[int]) -> List[int]:
        """One token per row of ``logits``; ``generated[i]`` is how many tokens row i's request
        has generated so far (the index of the token drawn now)."""
        return self.sample_async(logits, params, generated).tokens()

    def sample_async(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                     generated: Sequence[int]) -> SampledTokens:
        """As ``sample``, without waiting for the GPU."""
        if logits.shape[0] != len(params):
            raise ValueError("one row of logits per request")
        if logits.shape[0] == 0:
            return SampledTokens(torch.empty(0, dtype=torch.int32))
        if all(p.temperature <= 0 for p in params):
            ids = ops.sample(logits)
        else:
            temps = np.array([p.temperature for p in params], dtype=np.float32)
            us = np.array([uniform_for(p.seed, g) for p, g in zip(params, generated)],
                          dtype=np.float32)
            both = torch.from_numpy(np.stack([temps, us]))
            if logits.device.type == "cuda":
                both = both.pin_memory().to(logits.device, non_blocking=True)
            ids = ops.sample(logits, both[0].contiguous(), both[1].contiguous())
        return SampledTokens(ids)
