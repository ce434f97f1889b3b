"""The scheduler's decisions, on the CPU and without a model: token budget, order, the step
that turns a prompt into a running request, what happens when pages run out."""
import random

import pytest

from lucciola_amd.cache.manager import CacheManager
from lucciola_amd.cache.specs import PagedKV
from lucciola_amd.engine.scheduler import Scheduler
from lucciola_amd.engine.sequence import Sequence, SequenceStatus
from lucciola_amd.sampling.sampler import SamplingParams


def make(blocks=64, block_size=4, budget=16, max_seqs=8):
    cache = CacheManager([PagedKV(1, 16)], block_size, blocks, max_seqs)
    return Scheduler(cache, budget, max_seqs), cache


def run_step(sched, cache, step, token=7):
    """What the runner and the engine do with a scheduled step, minus the model."""
    for e in step.entries:
        if not cache.has(e.request):
            cache.admit(e.request)
        cache.reserve(e.request, len(e.tokens))
    for e in step.entries:
        cache.commit(e.request)
    finished = []
    for seq, samples in zip(step.seqs, step.samples):
        if samples and sched.on_token(seq, token):
            sched.free_sequence(seq)
            finished.append(seq)
    cache.check()
    return finished


def seq(i, n, new=4):
    return Sequence(i, list(range(1, n + 1)), SamplingParams(max_new_tokens=new))


def test_prompt_is_cut_under_the_budget_and_becomes_running():
    sched, cache = make(budget=16)
    s = seq(1, 40)
    sched.add_request(s)
    sizes = []
    while s.status is not SequenceStatus.RUNNING:
        step = sched.step()
        assert step.num_tokens <= 16 and step.num_prefill_seqs == 1 and step.num_decode_seqs == 0
        sizes.append(step.num_tokens)
        last = s.status is SequenceStatus.RUNNING
        assert step.samples == [last] and list(step.entries[0].want) == ([step.num_tokens - 1] if last else [])
        run_step(sched, cache, step)
    assert sizes == [16, 16, 8]
    assert s.get_len() == 41 and s.num_generated == 1     # that step's logits gave the first token
    step = sched.step()
    assert step.num_decode_seqs == 1 and step.entries[0].tokens == [7] and list(step.entries[0].want) == [0]


def test_decodes_come_first_and_count_against_the_budget():
    sched, cache = make(budget=8)
    a, b = seq(1, 3, new=50), seq(2, 3, new=50)
    sched.add_request(a)
    sched.add_request(b)
    run_step(sched, cache, sched.step())                  # both prompts fit one step
    assert a.status is b.status is SequenceStatus.RUNNING
    c = seq(3, 30)
    sched.add_request(c)
    step = sched.step()
    assert [e.request for e in step.entries] == [1, 2, 3]
    assert [len(e.tokens) for e in step.entries] == [1, 1, 6]     # 8 - 2 decodes
    assert step.num_decode_seqs == 2 and step.num_prefill_tokens == 6


def test_first_come_first_served_without_overtaking():
    sched, cache = make(blocks=10, block_size=4, budget=64)
    big, small = seq(1, 30, new=2), seq(2, 2, new=2)
    blocker = seq(3, 20, new=4)
    sched.add_request(blocker)
    run_step(sched, cache, sched.step())                  # holds 5 of 10 pages (6 after a token)
    sched.add_request(big)
    sched.add_request(small)
    step = sched.step()
    # the front request gets what fits (the portion is cut to the free pages); the one behind
    # it does not overtake
    ids = [e.request for e in step.entries]
    assert ids[0] == 3 and 2 not in ids
    if 1 in ids:
        assert len(step.entries[ids.index(1)].tokens) <= 4 * 4


def test_several_requests_start_in_one_step_and_max_seqs_holds():
    sched, cache = make(budget=64, max_seqs=3)
    for i in range(5):
        sched.add_request(seq(i + 1, 5))
    step = sched.step()
    assert [e.request for e in step.entries] == [1, 2, 3]
    run_step(sched, cache, step)
    assert len(sched.running) == 3 and len(sched.waiting) == 2


def test_requests_that_can_never_fit_are_refused():
    sched, cache = make(blocks=4, block_size=4)
    with pytest.raises(ValueError, match="exceed the cache"):
        sched.add_request(seq(1, 14, new=4))
    sched.max_model_len = 10
    with pytest.raises(ValueError, match="positions"):
        sched.add_request(seq(2, 8, new=4))
    with pytest.raises(ValueError):
        Sequence(3, [], SamplingParams())


def test_preemption_when_a_decode_finds_no_page():
    # the reference parks such a request for good (src/scheduler.cc:33-40); here it is fed again
    sched, cache = make(blocks=4, block_size=4, budget=32)
    a, b = seq(1, 8, new=8), seq(2, 8, new=8)
    sched.add_request(a)
    sched.add_request(b)
    run_step(sched, cache, sched.step())                  # 2 full pages each: the pool is full
    assert cache.groups[0].pool.num_free() == 0
    step = sched.step()                                   # both now need a third page
    assert step.preempted == [b]                          # the most recently admitted goes
    assert b.status is SequenceStatus.WAITING and b.prefill_offset == 0 and sched.waiting[0] is b
    assert not cache.has(2) and [e.request for e in step.entries] == [1]
    run_step(sched, cache, step)
    done = []
    for _ in range(200):
        if not sched.has_unfinished_requests():
            break
        step = sched.step()
        assert step.num_seqs > 0 or step.preempted
        done += run_step(sched, cache, step)
    assert {s.seq_id for s in done} == {1, 2}
    assert a.num_generated == 8 and b.num_generated == 8  # nothing lost, nothing emitted twice
    assert b.preemptions >= 1 and sched.num_preemptions >= 1
    assert cache.groups[0].pool.num_free() == 4 and not cache.requests


def test_a_preempted_request_feeds_what_it_generated_as_prompt():
    sched, cache = make(blocks=4, block_size=4, budget=32)
    a, b = seq(1, 8, new=8), seq(2, 8, new=8)
    sched.add_request(a)
    sched.add_request(b)
    run_step(sched, cache, sched.step(), token=50)
    step = sched.step()
    assert step.preempted == [b]
    run_step(sched, cache, step, token=51)
    assert b.token_ids[-1] == 50
    while not (a.is_finished()):
        step = sched.step()
        assert 2 not in [e.request for e in step.entries] or cache.groups[0].pool.num_free() > 0
        run_step(sched, cache, step, token=52)
    step = sched.step()
    entry = step.entries[[e.request for e in step.entries].index(2)]
    assert list(entry.tokens) == b.token_ids[:len(entry.tokens)] and entry.tokens[8] == 50


@pytest.mark.parametrize("seed", range(6))
def test_random_workloads_finish_and_give_everything_back(seed):
    rng = random.Random(seed)
    blocks, bs = rng.choice([(12, 4), (40, 2), (9, 8)])
    budget = rng.choice([8, 16, 33])
    sched, cache = make(blocks=blocks, block_size=bs, budget=budget, max_seqs=rng.choice([2, 4, 8]))
    pending = [Sequence(i + 1, [rng.randrange(100) for _ in range(rng.randint(1, blocks * bs // 3))],
                        SamplingParams(max_new_tokens=rng.randint(1, blocks * bs // 3)))
               for i in range(12)]
    done, steps = [], 0
    while pending or sched.has_unfinished_requests():
        if pending and rng.random() < 0.4:
            sched.add_request(pending.pop(0))
        if not sched.has_unfinished_requests():
            continue
        step = sched.step()
        steps += 1
        assert steps < 5000, "the scheduler does not make progress"
        assert step.num_tokens <= budget
        assert len({e.request for e in step.entries}) == len(step.entries)
        kinds = [len(e.tokens) == 1 and s.status is SequenceStatus.RUNNING and s.num_generated > 0
                 for e, s in zip(step.entries, step.seqs)]
        assert kinds == sorted(kinds, reverse=True)        # decodes before prompt portions
        for e in step.entries:
            assert cache.can_reserve(e.request if cache.has(e.request) else None, len(e.tokens))
        done += run_step(sched, cache, step, token=rng.randrange(100))
    assert len(done) == 12 and all(s.num_generated == s.params.max_new_tokens for s in done)
    assert cache.groups[0].pool.num_free() == blocks and not cache.requests


def test_portions_are_cut_at_the_multiple_a_mixer_asks_for():
    """A model whose mixer wants portions in multiples of 6: every portion but a prompt's last
    is one, under the budget and under the pages that are free; an undone step puts the
    portions back in their order."""
    cache = CacheManager([PagedKV(1, 16)], 4, 64, 8)
    sched = Scheduler(cache, 16, 8, portion_multiple=6)
    a, b = seq(1, 29), seq(2, 8)
    sched.add_request(a)
    sched.add_request(b)
    sizes = []
    while a.status is not SequenceStatus.RUNNING:
        step = sched.step()
        mine = [len(e.tokens) for e, s in zip(step.entries, step.seqs) if s is a]
        sizes += mine
        run_step(sched, cache, step)
    assert sizes == [12, 12, 5]                      # 16 cut down to 12; the last as it comes
    assert b.status is SequenceStatus.RUNNING        # 8 tokens were its whole prompt: no cut
    # undo: a step's portions wait again
    c, d = seq(3, 7), seq(4, 30)
    sched.add_request(c)
    sched.add_request(d)
    step = sched.step()
    assert [s.seq_id for s in step.seqs] == [1, 2, 3, 4] and step.portions == [0, 0, 7, 6]
    assert c.status is SequenceStatus.RUNNING and d.prefill_offset == 6
    sched.undo(step)
    assert [s.seq_id for s in sched.waiting] == [3, 4] and [s.seq_id for s in sched.running] == [1, 2]
    assert c.prefill_offset == 0 and d.prefill_offset == 0 and c.status is SequenceStatus.WAITING
    again = sched.step()
    assert [len(e.tokens) for e in again.entries] == [1, 1, 7, 6]
