"""The engine's host logic on the CPU: the step function, the cache and the batch layout are
run with the plain torch versions of the kernels put in their place, and compared with the
plain whole-sequence implementation.  What these tests cannot see is the kernels themselves
(the ``gpu`` tests cover those)."""

import pytest
import torch

import configs
import plain_qwen3
import reference_ops
import traces
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.engine.batch import StepEntry
from lucciola_amd.config.registry import architecture_for


from helpers import compare, make_runner, prompts_for, random_weights, replay


def make(cfg, seed, page, blocks, dtype="float32"):
    weights = random_weights(cfg, seed)
    return make_runner(cfg, weights, page, blocks, dtype, "cpu"), weights


@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_step_function_matches_plain(monkeypatch, key, family):
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL[key]
    lengths = {"A": [5, 11, 17, 40], "B": [1, 9, 30, 64, 45], "C": [70, 33, 50, 3, 61],
               "D": [37, 2, 50, 16]}[key]
    prompts = prompts_for(cfg, lengths, seed)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner, weights = make(cfg, seed, page, blocks)
    got = replay(runner, steps)
    assert len(got) == sum(lengths)
    compare(got, cfg, weights, prompts, 2e-5)
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


@pytest.mark.parametrize("key,page", [("C", 32), ("A", 48), ("D", 64)])
@pytest.mark.parametrize("family", ["chunked", "mixed"])
def test_pages_of_several_kernel_pages(monkeypatch, key, page, family):
    """A page of 32, 48 or 64 tokens goes to the kernels as two, three or four pages of 16 in a
    row: the cache counts in its own pages, the block tables on the device name the pieces."""
    reference_ops.install(monkeypatch)
    cfg, _, seed = configs.ALL[key]
    prompts = prompts_for(cfg, [70, 33, 50, 3, 131], seed)
    steps = {"chunked": traces.chunked, "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner, weights = make(cfg, seed, page, blocks)
    assert runner.cache.groups[0].kernel_page == 16 and runner.cache.groups[0].pieces == page // 16
    assert runner.cache.storage[0][0][0].shape[0] == blocks * (page // 16) and runner.cache.storage[0][0][0].shape[2] == 16
    got = replay(runner, steps)
    compare(got, cfg, weights, prompts, 2e-5)
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


def host_engine(cfg, weights, page, blocks, **kw):
    from lucciola_amd.engine.llm_engine import LLMEngine
    from lucciola_amd.engine.loading import _build
    from lucciola_amd.weights.loader import DictSource
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), "float32", "cpu")
    return LLMEngine(model, config, EngineConfig(dtype="float32", block_size=page,
                                                 max_blocks=blocks, device="cpu", **kw))


@pytest.mark.parametrize("blocks", [200, 11])
def test_running_ahead_generates_what_waiting_generates(monkeypatch, blocks):
    """A step queued before the tokens of the one before it are known, fed from the sampler's
    output: the same tokens as with a wait after every step, with plenty of pages and with so
    few that requests are preempted while a token of theirs is still under way."""
    from lucciola_amd.sampling.sampler import SamplingParams
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)
    prompts = list(prompts_for(cfg, [9, 14, 6, 11], seed + 40).values())
    params = [SamplingParams(max_new_tokens=n, temperature=t, seed=i)
              for i, (n, t) in enumerate([(20, 0.0), (1, 0.0), (17, 0.8), (2, 0.0)])]
    got = {}
    for ahead in (False, True):
        engine = host_engine(cfg, weights, page, blocks, max_tokens_per_step=12, max_seqs=4,
                             run_ahead=ahead)
        seen = []
        got[ahead] = engine.generate(prompts, params, on_token=lambda i, t, f: seen.append((i, t, f)))
        assert [len(g) for g in got[ahead]] == [20, 1, 17, 2]
        assert all(t >= 0 for g in got[ahead] for t in g)
        assert sum(f for _, _, f in seen) == 4 and len(seen) == 40
        if blocks == 11:
            assert engine.scheduler.num_preemptions > 0
        engine.runner.cache.check()
        assert not engine.runner.cache.requests and not engine.has_unfinished_requests()
    assert got[True] == got[False]
    assert got[False][0] == plain_qwen3.greedy(cfg, weights, prompts[0], 20)


def test_running_ahead_stops_at_an_end_token_and_drops_the_step_after_it(monkeypatch):
    from lucciola_amd.sampling.sampler import SamplingParams
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["B"]
    weights = random_weights(cfg, seed, std=0.3)
    prompts = list(prompts_for(cfg, [5, 12, 3], seed + 60).values())
    free_run = host_engine(cfg, weights, page, 64, max_seqs=4, run_ahead=False).generate(
        prompts, SamplingParams(max_new_tokens=12))
    stop = free_run[1][4]               # request 1 meets it at its fifth token at the latest
    want = []
    for tokens in free_run:
        cut = tokens.index(stop) + 1 if stop in tokens else len(tokens)
        want.append(tokens[:cut])
    assert len(want[1]) <= 5
    for ahead in (False, True):
        engine = host_engine(cfg, weights, page, 64, max_seqs=4, run_ahead=ahead)
        seen = []
        got = engine.generate(prompts, SamplingParams(max_new_tokens=12, eos_token_ids=(stop,)),
                              on_token=lambda i, t, f: seen.append((i, t, f)))
        assert got == want
        assert len(seen) == sum(len(w) for w in want) and sum(f for _, _, f in seen) == 3
        engine.runner.cache.check()
        assert not engine.runner.cache.requests
        for g in engine.runner.cache.groups:
            assert g.pool.num_free() == 64


def test_a_pending_token_needs_a_carry(monkeypatch):
    from lucciola_amd.engine.batch import PENDING, Carry
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["A"]
    runner, weights = make(cfg, seed, page, 32)
    logits = runner.step([StepEntry("a", [3, 4, 5], [2]), StepEntry("b", [7, 8], [1])])
    sampled = reference_ops.sample(logits)
    with pytest.raises(ValueError, match="no carry"):
        runner.step([StepEntry("a", [PENDING], [0])])
    with pytest.raises(ValueError, match="no row"):
        runner.step([StepEntry("a", [PENDING], [0])], Carry(sampled, {"b": 1}))
    with pytest.raises(ValueError, match="outside the vocabulary"):
        runner.step([StepEntry("a", [PENDING, 4], [0])], Carry(sampled, {"a": 0}))
    # one request fed from the device beside one fed from the host: as both from the host
    fed = runner.step([StepEntry("b", [int(sampled[1])], [0]), StepEntry("a", [PENDING], [0])],
                      Carry(sampled, {"a": 0, "b": 1}))
    ids = {"a": [3, 4, 5, int(sampled[0])], "b": [7, 8, int(sampled[1])]}
    for row, name in enumerate(["b", "a"]):
        ref = plain_qwen3.forward(cfg, weights, ids[name])[-1]
        assert float((fed[row].double() - ref).abs().max() / ref.abs().max()) < 2e-5


@pytest.mark.parametrize("ahead", [False, True])
def test_a_request_is_ended_early_and_gives_everything_back(monkeypatch, ahead):
    """Requests ended from outside while waiting, while their prompt is partly fed, and while
    running with a token under way: what they hold goes back at once, the others generate
    what they generate alone, and no token of an ended request comes out afterwards."""
    from lucciola_amd.sampling.sampler import SamplingParams
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)
    prompts = list(prompts_for(cfg, [9, 30, 6, 11], seed + 90).values())
    engine = host_engine(cfg, weights, page, 40, max_tokens_per_step=12, max_seqs=3, run_ahead=ahead)
    ids = [engine.add_request(p, SamplingParams(max_new_tokens=16)) for p in prompts]
    seen = {i: [] for i in ids}
    ended = set()
    steps = 0
    while engine.has_unfinished_requests():
        for out in engine.step():
            assert out.seq_id not in ended
            seen[out.seq_id].append(out.token)
        steps += 1
        if steps == 1:
            assert engine.abort_request(ids[3])                 # still waiting (max_seqs is 3)
            ended.add(ids[3])
        if steps == 2:
            assert 0 < engine.sequences[ids[1]].prefill_offset < 30
            assert engine.abort_request(ids[1])                 # its prompt is partly fed
            ended.add(ids[1])
        if steps == 6:
            assert engine.abort_request(ids[2])                 # running, a token may be under way
            ended.add(ids[2])
            assert not engine.abort_request(ids[2])
            engine.runner.cache.check()
            assert set(engine.runner.cache.requests) == {ids[0]}
    assert seen[ids[0]] == plain_qwen3.greedy(cfg, weights, prompts[0], 16)
    assert 0 < len(seen[ids[2]]) < 16 and seen[ids[1]] == [] and seen[ids[3]] == []
    assert seen[ids[2]] == plain_qwen3.greedy(cfg, weights, prompts[2], 16)[:len(seen[ids[2]])]
    assert all(t >= 0 for t in engine.sequences[ids[2]].token_ids)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests
    for g in engine.runner.cache.groups:
        assert g.pool.num_free() == 40
    assert not engine.abort_request(12345)


def test_a_step_that_raises_leaves_the_cache_and_the_queues_as_they_were(monkeypatch):
    """The model raises in the middle of a step (a kernel error, say): pages reserved for the
    step go back, a request that the step admitted leaves again, the scheduler's portions are
    waiting again, and the same work then runs to the plain implementation's tokens."""
    from lucciola_amd.sampling.sampler import SamplingParams
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)

    # the runner alone: a known request beside a new one
    runner = make_runner(cfg, weights, page, 16, "float32", "cpu")
    runner.step([StepEntry("a", [3, 4, 5, 6, 7], [4])])
    before = (runner.cache.length("a"), runner.cache.block_table(0, "a"), runner.cache.num_free_blocks())
    real_forward = runner.model.forward
    def broken(batch, sites):
        raise RuntimeError("injected")
    runner.model.forward = broken
    with pytest.raises(RuntimeError, match="injected"):
        runner.step([StepEntry("a", [8, 9, 10, 11, 12], [4]), StepEntry("b", [1, 2, 3], [2])])
    runner.cache.check()
    assert not runner.cache.has("b") and runner.cache.requests["a"].pending == 0
    assert (runner.cache.length("a"), runner.cache.block_table(0, "a"), runner.cache.num_free_blocks()) == before
    with pytest.raises(ValueError, match="outside its"):
        runner.step([StepEntry("a", [8, 9], [5])])       # raised while the batch is laid out
    runner.cache.check()
    assert runner.cache.requests["a"].pending == 0 and runner.cache.num_free_blocks() == before[2]
    runner.model.forward = real_forward
    got = runner.step([StepEntry("a", [8, 9, 10, 11, 12], [4])])[0].double()
    ref = plain_qwen3.forward(cfg, weights, [3, 4, 5, 6, 7, 8, 9, 10, 11, 12])[-1]
    assert float((got - ref).abs().max() / ref.abs().max()) < 2e-5

    # through the engine: the third step fails once, then everything goes on
    prompts = list(prompts_for(cfg, [9, 20, 6], seed + 7).values())
    engine = host_engine(cfg, weights, page, 40, max_tokens_per_step=12, max_seqs=3, run_ahead=False)
    ids = [engine.add_request(p, SamplingParams(max_new_tokens=6)) for p in prompts]
    real = engine.runner.model.forward
    calls = {"n": 0}
    def flaky(batch, sites):
        calls["n"] += 1
        if calls["n"] == 3:
            raise RuntimeError("injected")
        return real(batch, sites)
    engine.runner.model.forward = flaky
    seen = {i: [] for i in ids}
    failures = 0
    while engine.has_unfinished_requests():
        try:
            for out in engine.step():
                seen[out.seq_id].append(out.token)
        except RuntimeError:
            failures += 1
            engine.runner.cache.check()
            assert all(st.pending == 0 for st in engine.runner.cache.requests.values())
    assert failures == 1
    for i, p in zip(ids, prompts):
        assert seen[i] == plain_qwen3.greedy(cfg, weights, p, 6)
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_budgets_that_could_never_schedule_are_refused(monkeypatch):
    """A step budget below the multiple that the model's prompt portions must have is refused
    when the engine is made; a queue that holds requests none of which can ever run raises
    instead of spinning."""
    from lucciola_amd.sampling.sampler import SamplingParams
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)
    engine = host_engine(cfg, weights, page, 16, max_tokens_per_step=12, max_seqs=3)
    model = engine.model
    monkeypatch.setattr(type(model.layers[0].mixer), "portion_multiple", 16, raising=False)
    assert model.portion_multiple() == 16
    with pytest.raises(ValueError, match="below the 16 tokens"):
        host_engine(cfg, weights, page, 16, max_tokens_per_step=12, max_seqs=3)
    # a queue whose front request can never be cut into a portion (forced here past the check
    # above): the engine says so instead of scheduling nothing for ever
    monkeypatch.setattr(type(model.layers[0].mixer), "portion_multiple", 1, raising=False)
    for ahead in (False, True):
        engine = host_engine(cfg, weights, page, 16, max_tokens_per_step=12, max_seqs=3, run_ahead=ahead)
        engine.scheduler.portion_multiple = 16
        engine.add_request(list(range(40)), SamplingParams(max_new_tokens=2))
        with pytest.raises(RuntimeError, match="can run none of them"):
            engine.step()


def test_stats_say_where_the_host_time_went(monkeypatch):
    from lucciola_amd.sampling.sampler import SamplingParams
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)
    engine = host_engine(cfg, weights, page, 40, max_tokens_per_step=12, max_seqs=3, time_steps=True)
    engine.generate(list(prompts_for(cfg, [9, 20], seed).values()), SamplingParams(max_new_tokens=5))
    stats = engine.stats()
    for key in ("schedule_s", "reserve_s", "batch_s", "launch_s", "sample_s", "wait_s"):
        assert stats[key] > 0, key
    assert stats["steps"] > 5 and stats["graph_captures"] == 0
    assert stats["last_step_gpu_ms"] is None        # no device events on the CPU
