"""The engine: model runner + scheduler + sampler.

``LLMEngine.step`` is one turn of the reference's engine loop (src/async_engine.cc:113-160):
schedule, run the model, pick tokens, apply the stop rules, free what has finished.  The
reference waits for a step's tokens before it schedules the next.  Here the next step is
queued first (``EngineConfig.run_ahead``): the sampled ids stay on the device and feed the
next step from there, the host reads them one step late, and the GPU does not idle while the
host schedules.  What the host cannot know a step early is an end-of-sequence token: such a
request runs one step too many, whose token is thrown away.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence as Seq

import torch

from ..config.engine_config import EngineConfig
from ..sampling.sampler import Sampler, SamplingParams
from .batch import PENDING, Carry
from .loading import load_model, random_model
from .runner import ModelRunner
from .scheduler import ScheduledStep, Scheduler
from .sequence import Sequence


@dataclass
class StepOutput:
    seq_id: int
    token: int
    finished: bool


@dataclass
class _QueuedStep:
    """A step whose tokens the host has not read yet."""

    sampled: object                 # SampledTokens
    seqs: List[Sequence]            # the requests a token was sampled for, in row order
    places: List[int]               # where in each request's token list that token goes
    last: List[bool]                # the request reached max_new_tokens with this token
    events: Optional[tuple] = None  # (before, after) the step's kernels on the stream, when steps are timed


class LLMEngine:
    def __init__(self, model, model_config, engine_config: EngineConfig):
        self.model = model
        self.model_config = model_config
        self.config = engine_config
        multiple = model.portion_multiple()
        if engine_config.max_tokens_per_step < multiple:
            raise ValueError(f"max_tokens_per_step ({engine_config.max_tokens_per_step}) is below the "
                             f"{multiple} tokens that this model's prompt portions are multiples of: "
                             "no portion of a longer prompt could ever be scheduled")
        self.runner = ModelRunner(model, engine_config)
        self.scheduler = Scheduler(self.runner.cache, engine_config.max_tokens_per_step,
                                   engine_config.max_seqs,
                                   max_model_len=model.spec.max_positions,
                                   portion_multiple=model.portion_multiple())
        self.sampler = Sampler()
        self.sequences: Dict[int, Sequence] = {}
        self._next_id = 1
        self._queued: Optional[_QueuedStep] = None
        self.eos_token_ids = tuple(getattr(model_config, "eos_token_ids", ()) or ())
        # seconds of host time by what they went to (the runner keeps its own for the step itself)
        self.times = {"schedule": 0.0, "sample": 0.0, "wait": 0.0}
        self.last_step_gpu_ms: Optional[float] = None

    @classmethod
    def from_folder(cls, model_path: str, engine_config: Optional[EngineConfig] = None):
        engine_config = engine_config or EngineConfig()
        model, cfg = load_model(model_path, engine_config.dtype, engine_config.device)
        return cls(model, cfg, engine_config)

    @classmethod
    def from_random(cls, config_dict, seed: int, engine_config: Optional[EngineConfig] = None):
        engine_config = engine_config or EngineConfig()
        model, cfg = random_model(config_dict, seed, engine_config.dtype, engine_config.device)
        return cls(model, cfg, engine_config)

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt_token_ids: Seq[int], params: Optional[SamplingParams] = None) -> int:
        params = params or SamplingParams()
        if not params.eos_token_ids and self.eos_token_ids:
            params.eos_token_ids = self.eos_token_ids
        V = self.model.vocab_size
        for t in prompt_token_ids:
            if not 0 <= int(t) < V:
                raise ValueError(f"token id {t} is outside the vocabulary of {V}")
        seq = Sequence(self._next_id, prompt_token_ids, params)
        self._next_id += 1
        self.scheduler.add_request(seq)
        self.sequences[seq.seq_id] = seq
        return seq.seq_id

    def abort_request(self, seq_id: int) -> bool:
        """End a request now, wherever it is (waiting, partly fed, running, with a token under
        way): its pages and its slot go back, tokens that the host has not read yet are
        dropped.  Returns False if there is no such live request."""
        seq = self.sequences.get(seq_id)
        if seq is None or seq.is_finished():
            return False
        while seq.get_len() > seq.get_prompt_len() and seq.token_ids[-1] == PENDING:
            seq.token_ids.pop()        # `_collect` skips a place beyond the request's end
        self.scheduler.free_sequence(seq)
        return True

    def has_unfinished_requests(self) -> bool:
        return self._queued is not None or self.scheduler.has_unfinished_requests()

    # ------------------------------------------------------------------ one step
    def step(self) -> List[StepOutput]:
        """Queue the next step, then hand out the tokens of the step queued before it (without
        ``run_ahead``: of this very step)."""
        if not self.config.run_ahead:
            only = self._launch(None)
            return self._collect(only) if only is not None else []
        before = self._queued
        self._queued = self._launch(before)
        if before is None:
            if self._queued is None:
                return []
            # nothing was in flight: queue a second step, so that from now on one is always
            # running while the host reads the tokens of the one before
            before = self._queued
            self._queued = self._launch(before)
        return self._collect(before)

    def _launch(self, before: Optional[_QueuedStep]) -> Optional[_QueuedStep]:
        """Schedule and queue one step.  Requests whose last token is still on the device
        (sampled by ``before``) are fed from there."""
        t_in = time.perf_counter()
        sched: ScheduledStep = self.scheduler.step()
        self.times["schedule"] += time.perf_counter() - t_in
        if sched.num_seqs == 0:
            if before is None and self.scheduler.has_unfinished_requests() and not sched.preempted:
                raise RuntimeError("the scheduler has requests but can run none of them")
            return None
        carry = None
        if before is not None and before.sampled is not None:
            carry = Carry(before.sampled.ids, {s.seq_id: row for row, s in enumerate(before.seqs)})
        events = None
        if self.config.time_steps and self.runner.device.type == "cuda":
            events = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            events[0].record()
        try:
            logits = self.runner.step(sched.entries, carry)
        except BaseException:
            self.scheduler.undo(sched)      # the runner has put the cache back as it was
            raise
        sampling = [seq for seq, s in zip(sched.seqs, sched.samples) if s]
        if not sampling:
            if events is not None:
                events[1].record()
            return _QueuedStep(None, [], [], [], events)
        t_in = time.perf_counter()
        sampled = self.sampler.sample_async(logits, [s.params for s in sampling],
                                            [s.num_generated for s in sampling])
        self.times["sample"] += time.perf_counter() - t_in
        if events is not None:
            events[1].record()
        places, last = [], []
        for seq in sampling:
            places.append(seq.get_len())
            done = self.scheduler.on_token(seq, PENDING)    # the count is known, the token is not
            if done:
                self.scheduler.free_sequence(seq)
            last.append(done)
        return _QueuedStep(sampled, sampling, places, last, events)

    def _collect(self, step: _QueuedStep) -> List[StepOutput]:
        """Read a queued step's tokens, put them where they belong and apply the stop rules
        that need the token itself."""
        outputs: List[StepOutput] = []
        if step.sampled is None:
            return outputs
        t_in = time.perf_counter()
        tokens = step.sampled.tokens()          # waits until the step's ids have reached the host
        self.times["wait"] += time.perf_counter() - t_in
        if step.events is not None:
            step.events[1].synchronize()
            self.last_step_gpu_ms = step.events[0].elapsed_time(step.events[1])
        for seq, place, last, token in zip(step.seqs, step.places, step.last, tokens):
            if place >= seq.get_len():
                continue        # the request ended on an earlier token: this one is thrown away
            seq.token_ids[place] = token
            finished = last
            if not finished and seq.stops_on(token):
                del seq.token_ids[place + 1:]       # a token queued after the last one
                self.scheduler.free_sequence(seq)
                finished = True
            outputs.append(StepOutput(seq.seq_id, token, finished))
        return outputs

    def stats(self) -> Dict[str, float]:
        """Counters (steps and tokens run, graph replays and captures, preemptions, pages and
        slots in use) and where the host's time went, in seconds since the engine was made:
        ``schedule_s`` deciding the steps, ``reserve_s`` checking entries and taking pages,
        ``batch_s`` laying out batches and sending them, ``launch_s`` queueing the model's
        kernels or replaying captured steps, ``sample_s`` queueing the sampler, ``wait_s``
        waiting for a step's tokens to reach the host (with ``run_ahead`` the GPU works on the
        next step meanwhile).  ``last_step_gpu_ms``: the time between two events around the
        last step whose tokens were read, when ``EngineConfig.time_steps`` is set (the
        reference brackets its runs with events the same way, benchmarks/basic_bench.cc:27-64)."""
        cache, runner = self.runner.cache, self.runner
        return {
            "steps": runner.steps, "tokens": runner.tokens,
            "graph_replays": runner.graph_replays, "graph_captures": runner.graph_captures,
            "preemptions": self.scheduler.num_preemptions,
            "waiting": len(self.scheduler.waiting), "running": len(self.scheduler.running),
            "pages_total": cache.num_blocks, "pages_free": cache.num_free_blocks(),
            "slots_free": cache.slots.num_free(),
            "schedule_s": self.times["schedule"], "reserve_s": runner.times["reserve"],
            "batch_s": runner.times["batch"], "launch_s": runner.times["launch"],
            "sample_s": self.times["sample"], "wait_s": self.times["wait"],
            "last_step_gpu_ms": self.last_step_gpu_ms,
        }

    # ------------------------------------------------------------------ whole requests
    def generate(self, prompts: Seq[Seq[int]], params=None,
                 on_token: Optional[Callable[[int, int, bool], None]] = None) -> List[List[int]]:
        """Generate for every prompt (lists of token ids); returns the generated ids of each."""
        if params is None or isinstance(params, SamplingParams):
            params = [params] * len(prompts)
        ids = []
        for prompt, p in zip(prompts, params):
            p = SamplingParams(**vars(p)) if p is not None else None
            ids.append(self.add_request(prompt, p))
        while self.has_unfinished_requests():
            for out in self.step():
                if on_token is not None:
                    on_token(out.seq_id, out.token, out.finished)
        result = [self.sequences[i].output_token_ids for i in ids]
        for i in ids:
            del self.sequences[i]
        return result
