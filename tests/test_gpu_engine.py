"""The engine on the GPU against the plain implementation, in float32 and in bfloat16: each
request alone and whole; most of it in one step and the last 32 tokens one by one; portions of
changing size; mixed batches with so few pages that they are used again; long decoding; the
first tokens of a sequence; generation through the entry points; trace replay."""
import json
import os
import subprocess
import sys

import pytest
import torch

import configs
import plain_qwen3
import traces
from helpers import compare, make_runner, prompts_for, random_weights, replay
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.engine.llm_engine import LLMEngine
from lucciola_amd.engine.loading import _build
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.sampling.sampler import SamplingParams, uniform_for
from lucciola_amd.weights.loader import DictSource
from lucciola_amd.weights.random_init import write_model_folder

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# error of a row of logits: max |difference| / max |logit|
TOL = {"float32": 2e-5, "bfloat16": 3e-2}
LENGTHS = {"A": [5, 11, 17, 40, 130], "B": [1, 9, 30, 64, 45, 200], "C": [70, 33, 50, 3, 61, 150],
           "D": [37, 2, 90, 16, 140]}

_cache = {}


def case(key):
    if key not in _cache:
        cfg, page, seed = configs.ALL[key]
        weights = random_weights(cfg, seed)
        prompts = prompts_for(cfg, LENGTHS[key], seed)
        refs = {n: plain_qwen3.forward(cfg, weights, ids) for n, ids in prompts.items()}
        _cache[key] = (cfg, page, weights, prompts, refs)
    return _cache[key]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_replay_families(dtype, key, family):
    cfg, page, weights, prompts, refs = case(key)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
    got = replay(runner, steps)
    assert len(got) == sum(len(p) for p in prompts.values())
    worst = compare(got, cfg, weights, prompts, TOL[dtype], refs)
    print(f"{key} {family} {dtype}: worst relative error {worst:.3e}")
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key,page", [("C", 32), ("A", 48), ("D", 64), ("D", 32)])
def test_pages_of_several_kernel_pages(dtype, key, page):
    """Pages of 32, 48 and 64 tokens, which the kernels see as runs of pages of 16: mixed with
    so few pages that they are used again, and with a decoded tail.  (D's heads of 64 go
    through the matrix-core kernels in bfloat16.)"""
    cfg, _, seed = configs.ALL[key]
    weights = random_weights(cfg, seed)
    prompts = prompts_for(cfg, [70, 33, 150, 3, 131], seed + 5)
    refs = {n: plain_qwen3.forward(cfg, weights, ids) for n, ids in prompts.items()}
    for family in (traces.mixed, traces.tail_decode):
        steps = family(prompts)
        blocks = traces.max_live_tokens(steps, page) // page
        runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
        assert runner.cache.groups[0].pieces == page // 16
        got = replay(runner, steps)
        assert len(got) == sum(len(p) for p in prompts.values())
        compare(got, cfg, weights, prompts, TOL[dtype], refs)
        for g in runner.cache.groups:
            assert g.pool.num_free() == blocks


def random_configuration(seed):
    """A configuration drawn at random from what config.json allows: any number of heads and
    groups, head sizes in steps of 16, widths, feed-forward sizes and vocabularies that are odd
    or not, windows on some layers, any page size."""
    import random
    rng = random.Random(1000 + seed)
    layers = rng.randint(1, 4)
    kv = rng.choice([1, 2, 3, 4])
    group = rng.choice([1, 2, 3, 4, 5, 6, 8])
    cfg = {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
        "num_hidden_layers": layers, "hidden_size": rng.choice([24, 40, 75, 100, 128, 136, 200, 256]),
        "num_attention_heads": kv * group, "num_key_value_heads": kv,
        "head_dim": rng.choice([16, 32, 48, 64, 80, 96, 112, 128]),
        "intermediate_size": rng.choice([16, 57, 88, 128, 130, 256, 301, 384]),
        "vocab_size": rng.randint(50, 700),
        "rope_theta": rng.choice([10000.0, 50000.0, 1000000.0]),
        "rms_norm_eps": rng.choice([1e-6, 3e-6, 1e-5]),
        "tie_word_embeddings": rng.random() < 0.5, "max_position_embeddings": 4096,
        "initializer_range": rng.choice([0.02, 0.05]), "hidden_act": "silu",
    }
    if rng.random() < 0.5:
        cfg["sliding_window"] = rng.randint(5, 40)
        cfg["use_sliding_window"] = True
        cfg["layer_types"] = [rng.choice(["full_attention", "sliding_attention"]) for _ in range(layers)]
        if "sliding_attention" not in cfg["layer_types"]:
            cfg["layer_types"][rng.randrange(layers)] = "sliding_attention"
    page = rng.choice([4, 8, 16, 32])
    lengths = [rng.randint(1, 150) for _ in range(5)]
    return cfg, page, lengths


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(seed, dtype):
    """Configurations drawn at random, replayed mixed (pages used again) and with a decoded
    tail: sizes that no fixed test names must give right results too, through whichever kernel
    takes them."""
    cfg, page, lengths = random_configuration(seed)
    weights = random_weights(cfg, seed)
    prompts = prompts_for(cfg, lengths, seed)
    refs = {n: plain_qwen3.forward(cfg, weights, ids) for n, ids in prompts.items()}
    for family in (traces.mixed, traces.tail_decode):
        steps = family(prompts)
        blocks = traces.max_live_tokens(steps, page) // page
        runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
        got = replay(runner, steps)
        assert len(got) == sum(len(p) for p in prompts.values())
        worst = compare(got, cfg, weights, prompts, TOL[dtype], refs)
        print(f"seed {seed} {family.__name__} {dtype}: {cfg['num_attention_heads']} heads of "
              f"{cfg['head_dim']} in {cfg['num_key_value_heads']} groups, width {cfg['hidden_size']}, "
              f"page {page}: worst relative error {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_reused_with_stale_contents(dtype):
    """Requests run one after the other in a pool that holds only one of them, after the pool
    has been filled with large values: what a page held before must never show."""
    cfg, page, weights, prompts, refs = case("B")
    steps = traces.chunked(prompts, sizes=(9, 2, 30))
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
    for ((k, v),) in runner.cache.storage.values():
        k.fill_(300.0)
        v.fill_(-300.0)
    compare(replay(runner, steps), cfg, weights, prompts, TOL[dtype], refs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "C"])
def test_long_decoding(dtype, key):
    cfg, page, seed = configs.ALL[key]
    weights = random_weights(cfg, seed)
    prompts = prompts_for(cfg, [700], seed + 10)
    steps = traces.tail_decode(prompts, tail=660)
    runner = make_runner(cfg, weights, page, -(-700 // page), dtype, DEV)
    compare(replay(runner, steps, check=False), cfg, weights, prompts, TOL[dtype])


# narrow models whose heads the matrix-core attention kernels take: heads of 128 (two to a kv
# head) and heads of 64 (three kv heads)
LONG_128 = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 256, "vocab_size": 211,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": False,
    "max_position_embeddings": 4096, "initializer_range": 0.05, "hidden_act": "silu",
}
LONG_64 = dict(configs.TINY_D, max_position_embeddings=4096)


def peaked(weights, factor=2.0):
    """The same weights with every q norm scaled up: with the q/k norms the scores of random
    weights have a spread of about one whatever the projections are, so every key counts about
    the same and one page left out among a hundred would move the result by a hundredth.
    Scaled, a few keys anywhere in the context carry a row's weight, and a key that is read
    wrongly or not at all shows."""
    return {n: (t.float() * factor).to(t.dtype) if n.endswith("q_norm.weight") else t
            for n, t in weights.items()}


@pytest.mark.parametrize("cfg", [LONG_128, LONG_64], ids=["heads128", "heads64"])
def test_long_decoding_through_captured_steps(cfg):
    """bfloat16 decoding from 900 to 2,260 tokens through the matrix-core attention, as the
    engine serves it: steps replayed from HIP graphs, whose block tables widen twice on the way
    (64, 128 and 192 pages of 16), with a request's pages cut into shares that a second kernel
    joins; every position against the plain implementation."""
    from lucciola_amd.kernels import ops
    page, total, cut = 16, 2260, 900
    weights = peaked(random_weights(cfg, 21))
    prompts = prompts_for(cfg, [total], 22)
    steps = traces.tail_decode(prompts, tail=total - cut)
    runner = make_runner(cfg, weights, page, -(-total // page), "bfloat16", DEV)
    assert runner.use_graphs
    got = replay(runner, steps, check=False)
    assert runner.graph_replays >= total - cut - 3 and runner.graph_captures == 3
    assert sorted(k[1] for k in runner._graphs) == [64, 128, 192]
    nkv = cfg["num_key_value_heads"]
    for pad in (64, 128, 192):
        assert ops.library().lc_attn_decode_splits(1, nkv, pad * page) > 1
    worst = compare(got, cfg, weights, prompts, TOL["bfloat16"])
    print(f"long decoding, heads of {cfg['head_dim']}: worst relative error {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
def test_first_tokens(dtype, key):
    cfg, page, seed = configs.ALL[key]
    weights = random_weights(cfg, seed)
    prompts = prompts_for(cfg, [1, 2, 3, 4], seed + 20)
    for family in (traces.whole, lambda p: traces.tail_decode(p, tail=3)):
        runner = make_runner(cfg, weights, page, 8, dtype, DEV)
        compare(replay(runner, family(prompts)), cfg, weights, prompts, TOL[dtype])


def engine_for(cfg, weights, page, blocks, dtype, **kw):
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), dtype, DEV)
    return LLMEngine(model, config, EngineConfig(dtype=dtype, block_size=page, max_blocks=blocks,
                                                 device=DEV, **kw))


@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
def test_greedy_generation_through_the_engine(key):
    cfg, page, seed = configs.ALL[key]
    weights = random_weights(cfg, seed, std=0.3)
    prompts = list(prompts_for(cfg, [5, 11, 17], seed + 30).values())
    engine = engine_for(cfg, weights, page, 64, "float32", max_tokens_per_step=16, max_seqs=4)
    got = engine.generate(prompts, SamplingParams(max_new_tokens=8))
    want = [plain_qwen3.greedy(cfg, weights, p, 8) for p in prompts]
    assert got == want
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


@pytest.mark.parametrize("ahead", [False, True])
def test_generation_survives_preemption(ahead):
    """With so few pages that running requests are preempted and recomputed, every request's
    tokens are those of the plain implementation (greedy ones, and the temperature draws too:
    a draw depends on the request's seed and the token's index alone)."""
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)
    prompts = list(prompts_for(cfg, [9, 14, 6, 11], seed + 40).values())
    tight = engine_for(cfg, weights, page, 18, "float32", max_tokens_per_step=12, max_seqs=4,
                       run_ahead=ahead)
    got = tight.generate(prompts, SamplingParams(max_new_tokens=20))
    assert tight.scheduler.num_preemptions > 0
    for prompt, tokens in zip(prompts, got):
        assert tokens == plain_qwen3.greedy(cfg, weights, prompt, 20)
    tight.runner.cache.check()
    assert not tight.runner.cache.requests
    params = [SamplingParams(max_new_tokens=20, temperature=0.7 if i % 2 else 0.0, seed=50 + i)
              for i in range(4)]
    got = tight.generate(prompts, params)
    assert tight.scheduler.num_preemptions > 1
    for prompt, p, tokens in zip(prompts, params, got):
        check_sampled(cfg, weights, prompt, p, tokens)


def record_logits(engine):
    """Keep every row of logits that ``engine`` samples from, by (the request's params object,
    index of the token drawn): ``generate`` gives every request a params object of its own."""
    rows = {}
    inner = engine.sampler.sample_async

    def sample_async(logits, params, generated):
        kept = logits.double().cpu()
        for r, (p, g) in enumerate(zip(params, generated)):
            rows[(id(p), g)] = kept[r]
        return inner(logits, params, generated)
    engine.sampler.sample_async = sample_async
    return rows


def generate_recorded(engine, prompts, params):
    """What ``engine.generate`` does, keeping the logits of every token it sampled: the
    generated tokens and {request index: rows} (``rows[i]`` is the row token i was drawn from)."""
    if isinstance(params, SamplingParams):
        params = [params] * len(prompts)
    own = [SamplingParams(**vars(p)) for p in params]
    kept = record_logits(engine)
    ids = [engine.add_request(prompt, p) for prompt, p in zip(prompts, own)]
    while engine.has_unfinished_requests():
        engine.step()
    out = [engine.sequences.pop(i).output_token_ids for i in ids]
    rows = [[kept[(id(p), i)] for i in range(len(tokens))] for tokens, p in zip(out, own)]
    return out, rows


def check_sampled(cfg, weights, prompt, params, tokens, rows=None):
    """Every token of a request against the plain implementation's pick at its place.

    Without ``rows`` (float32) a pick may differ only at a boundary of the cumulative
    distribution (1e-4).  With ``rows`` (bfloat16: the logits the engine sampled each token
    from) the row's own measured error e = max |row - plain row| decides what rounding can
    explain: a greedy pick must lie within 2 e of the top, and a draw may fall to the other
    side of a boundary only if that boundary, at cumulative probability c, lies within
    c (1 - c) (exp(2 e / T) - 1) of the uniform number: as far as errors of at most e in every
    logit can move it."""
    logits_all = plain_qwen3.forward(cfg, weights, list(prompt) + list(tokens))
    for i, tok in enumerate(tokens):
        logits = logits_all[len(prompt) - 1 + i]
        err = 0.0
        if rows is not None:
            err = float((rows[i] - logits).abs().max())
            # (these tests use weights of ten times the usual spread, so that picks are decided:
            # their rows' errors reach 4e-2 of the largest logit, and were allowed 6e-2 before
            # each pick was held against its own row)
            assert err <= 6e-2 * float(logits.abs().max()), (i, err)
        u = uniform_for(params.seed, i)
        want = plain_qwen3.sample_token(logits, params.temperature, u)
        if tok == want:
            continue
        if params.temperature > 0:    # only a rounding neighbour of the CDF boundary may differ
            pr = torch.softmax(logits / params.temperature, 0).cumsum(0)
            lo, hi = min(tok, want), max(tok, want)
            # every boundary between the two picks must be one that the errors can move past u
            for b in range(lo, hi):
                c = float(pr[b])
                allowed = 1e-4 if rows is None else c * (1 - c) * (float(torch.exp(torch.tensor(2 * err / params.temperature))) - 1) + 1e-6
                assert abs(c - u) <= allowed, (i, tok, want, c, u, allowed)
        else:
            assert float(logits.max() - logits[tok]) <= 2 * err + 1e-9, (i, tok, want, err)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    cfg, page, seed = configs.ALL["C"]
    folder = write_model_folder(str(tmp_path / "model"), cfg, seed)
    from lucciola_amd.weights.safetensors_io import SafetensorsFile
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        weights = {n: f.get(n).clone() for n in f.names()}
    prompts = prompts_for(cfg, [70, 33, 50, 3, 61], seed)
    steps = traces.mixed(prompts, seed=3)
    lines, index = [], {}
    fed = {}
    for i, (entries, end) in enumerate(steps):
        lines.append(json.dumps({"step": i, "end": end, "entries": [
            {"id": n, "tokens": t, "want": w} for n, t, w in entries]}))
        rows = []
        for n, t, w in entries:
            rows += [(n, fed.get(n, 0) + k) for k in w]
            fed[n] = fed.get(n, 0) + len(t)
        index[i] = rows
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder,
                           "--dtype", dtype, "--out", str(out), "--max-tokens",
                           str(traces.max_live_tokens(steps, 64))],
                          input="\n".join(lines) + "\n", text=True, capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [x for i in range(len(steps)) for x in ("done", str(i))]
    import numpy as np
    got = {}
    for i, rows in index.items():
        if not rows:
            assert not (out / f"{i}.f32").exists()
            continue
        data = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(len(rows), cfg["vocab_size"])
        for r, key in enumerate(rows):
            got[key] = torch.from_numpy(data[r].astype("float64"))
    compare(got, cfg, weights, prompts, TOL[dtype])


def test_graph_replay_matches_eager():
    """Decode steps replayed from a captured HIP graph, with eager steps (prompt portions of
    other requests, synchronisations) between the replays: every replay gives the logits of an
    engine that never uses graphs."""
    cfg, page, seed = configs.ALL["C"]
    weights = random_weights(cfg, seed)
    prompts = prompts_for(cfg, [40, 75, 20], seed + 60)
    extra = prompts_for(cfg, [90], seed + 61)["r0"]
    results = {}
    for use_graphs in (False, True):
        arch = architecture_for(cfg)
        model = _build(arch.model_spec(arch.read_config(cfg)), DictSource(weights), "bfloat16", DEV)
        from lucciola_amd.engine.runner import ModelRunner
        from lucciola_amd.engine.batch import StepEntry
        runner = ModelRunner(model, EngineConfig(dtype="bfloat16", block_size=page, max_blocks=64,
                                                 max_seqs=8, device=DEV, use_graphs=use_graphs))
        rows = []
        for name, ids in prompts.items():
            runner.step([StepEntry(name, ids[:10], [])])
        fed = {name: 10 for name in prompts}
        for step in range(10):
            entries = [StepEntry(n, [prompts[n][fed[n]]], [0]) for n in prompts]
            rows.append(runner.step(entries).float().cpu())
            for n in prompts:
                fed[n] += 1
            if step % 3 == 1:      # eager work between replays
                runner.step([StepEntry("extra", extra[step * 5:step * 5 + 5], [4])])
                torch.cuda.synchronize()
        results[use_graphs] = torch.stack(rows)
        if use_graphs:
            assert runner.graph_replays >= 8
        else:
            assert runner.graph_replays == 0
    assert torch.equal(results[True], results[False])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "D"])
def test_running_ahead_matches_waiting(dtype, key):
    """The engine queues a step before it has read the tokens of the one before (they reach the
    next step on the device).  With requests that end at different times, by count and by an
    end token, with temperature beside greedy, through eager steps (float32) and graph replays
    (bfloat16): the same tokens as an engine that waits after every step (float32), the plain
    implementation's tokens (both)."""
    cfg, page, seed = configs.ALL[key]
    weights = random_weights(cfg, seed, std=0.3)
    prompts = list(prompts_for(cfg, [9, 14, 6, 11, 3], seed + 80).values())
    counts = [24, 1, 17, 2, 30]
    got, rows = {}, {}
    stop = None
    for ahead in (False, True):
        engine = engine_for(cfg, weights, page, 256 // page + 8, dtype, max_tokens_per_step=12,
                            max_seqs=5, run_ahead=ahead)
        if stop is None:        # an end token that request 4 meets half way
            stop = engine.generate([prompts[4]], SamplingParams(max_new_tokens=30))[0][14]
        params = [SamplingParams(max_new_tokens=n, temperature=0.7 if i == 2 else 0.0, seed=i,
                                 eos_token_ids=(stop,) if i == 4 else ())
                  for i, n in enumerate(counts)]
        got[ahead], rows[ahead] = generate_recorded(engine, prompts, params)
        assert [len(g) for g in got[ahead]][:4] == counts[:4]
        last = got[ahead][4]
        assert stop not in last[:-1] and (last[-1] == stop or len(last) == 30)
        if dtype == "float32":
            assert last[-1] == stop and len(last) <= 15
        engine.runner.cache.check()
        assert not engine.runner.cache.requests
        if dtype == "bfloat16":
            assert engine.runner.graph_replays > 10
    if dtype == "float32":
        assert got[True] == got[False]
    # every request against the plain implementation (in bfloat16 the step after an end token
    # holds a row more when running ahead, other kernels may compute it, and a close pick may
    # fall the other way: both ways are checked, with bfloat16's allowance)
    for way in ([True] if dtype == "float32" else [False, True]):
        for prompt, p, tokens, kept in zip(prompts, params, got[way], rows[way]):
            check_sampled(cfg, weights, prompt, p, tokens, rows=None if dtype == "float32" else kept)


@pytest.mark.parametrize("trial", list(range(12)) + [16, 23, 129, 204])
def test_running_ahead_under_random_workloads(trial):
    """Random requests (lengths, counts, end tokens, temperature), budgets and pool sizes, some so
    tight that requests are preempted: running ahead and waiting generate the same in float32,
    and in both dtypes what the plain implementation picks (trials 16, 23, 129 and 204 are ones where
    bfloat16 rounding makes the two ways differ)."""
    import random
    rng = random.Random(1000 + trial)
    cfg, page, seed = configs.ALL[rng.choice("ABCD")]
    dtype = rng.choice(["float32", "bfloat16"])
    weights = random_weights(cfg, seed + trial, std=0.3)
    n = rng.randint(2, 6)
    prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(1, 40))] for _ in range(n)]
    counts = [rng.randint(1, 30) for _ in range(n)]
    eos = tuple(rng.sample(range(cfg["vocab_size"]), 12))
    roomy = sum(len(p) + c for p, c in zip(prompts, counts)) // page + n + 2
    tight = max((len(p) + c) // page + 2 for p, c in zip(prompts, counts)) + rng.randint(1, 6)
    blocks, budget = rng.choice([roomy, tight]), rng.choice([8, 16, 64])
    got, rows = {}, {}
    for ahead in (False, True):
        engine = engine_for(cfg, weights, page, blocks, dtype, max_tokens_per_step=budget, max_seqs=4,
                            run_ahead=ahead)
        params = [SamplingParams(max_new_tokens=c, temperature=0.8 if i % 3 == 1 else 0.0, seed=i,
                                 eos_token_ids=eos if i % 2 == 0 else ()) for i, c in enumerate(counts)]
        got[ahead], rows[ahead] = generate_recorded(engine, prompts, params)
        engine.runner.cache.check()
        assert not engine.runner.cache.requests
    if dtype == "float32":
        assert got[True] == got[False]
    # in bfloat16 the two ways put other rows side by side in a step, other kernels compute the
    # products, and a pick between two tokens that are close may fall the other way: each way is
    # checked against the plain implementation along what it generated
    for way in ([True] if dtype == "float32" else [False, True]):
        for prompt, p, count, tokens, kept in zip(prompts, params, counts, got[way], rows[way]):
            assert 1 <= len(tokens) <= count
            assert all(tok not in p.eos_token_ids for tok in tokens[:-1])
            assert len(tokens) == count or tokens[-1] in p.eos_token_ids
            check_sampled(cfg, weights, prompt, p, tokens, rows=None if dtype == "float32" else kept)


def test_command_line_and_async_engine(tmp_path):
    """The command line and ``AsyncEngine(model_path, max_blocks, block_size)`` /
    ``generate_async(prompt, max_new_tokens, callback)`` give the plain greedy tokens."""
    import threading
    from lucciola_amd import AsyncEngine
    from lucciola_amd.weights.safetensors_io import SafetensorsFile
    cfg, page, seed = configs.ALL["B"]
    folder = write_model_folder(str(tmp_path / "model"), cfg, seed, std=0.3)
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        weights = {n: f.get(n).clone() for n in f.names()}
    prompts = list(prompts_for(cfg, [4, 13], seed + 70).values())
    want = [plain_qwen3.greedy(cfg, weights, p, 6) for p in prompts]

    cmd = [sys.executable, "-m", "lucciola_amd", "--model", folder, "--dtype", "float32",
           "--max-blocks", "32", "--block-size", str(page), "--max-new-tokens", "6"]
    for p in prompts:
        cmd += ["--prompt-ids", ",".join(map(str, p))]
    proc = subprocess.run(cmd + ["--stats"], cwd=ROOT, text=True, capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [[int(t) for t in line.split()] for line in proc.stdout.strip().splitlines()] == want
    stats = json.loads(proc.stderr.strip().splitlines()[-1])       # --stats: the last line on standard error
    assert stats["steps"] >= 6 and stats["launch_s"] > 0 and stats["last_step_gpu_ms"] > 0
    # interactive: a request per line until "exit"
    proc = subprocess.run(cmd[:cmd.index("--prompt-ids")], cwd=ROOT, text=True, capture_output=True,
                          timeout=600, input=" ".join(map(str, prompts[0])) + "\nexit\n")
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == want[0]

    # text: a vocab.json beside the weights (every byte a token), the chat format with ids of this vocabulary
    from lucciola_amd.text.vocab_tokenizer import ChatFormat, VocabTokenizer, byte_alphabet
    vocab = {c: b for b, c in enumerate(byte_alphabet())}
    with open(os.path.join(folder, "vocab.json"), "w", encoding="utf-8") as fh:
        json.dump(vocab, fh)
    tok, fmt = VocabTokenizer(vocab), ChatFormat(380, 381, 382)
    text_prompt = fmt.prompt(tok, "hi there")
    text_want = tok.decode(plain_qwen3.greedy(cfg, weights, text_prompt, 6))
    text_cmd = cmd[:cmd.index("--prompt-ids")] + ["--chat-ids", "380,381,382"]
    utf8 = dict(os.environ, PYTHONUTF8="1")          # bytes, not text: random tokens hold line ends of every kind
    proc = subprocess.run(text_cmd + ["--prompt", "hi there"], cwd=ROOT, capture_output=True, timeout=600, env=utf8)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout == (text_want + "\n").encode("utf-8")
    proc = subprocess.run(text_cmd + ["--text"], cwd=ROOT, capture_output=True, timeout=600, env=utf8,
                          input=b"hi there\nexit\n")
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout == (text_want + "\n").encode("utf-8")

    engine = AsyncEngine(folder, max_blocks=32, block_size=page, dtype="float32")
    assert engine.tokenizer is not None and len(engine.tokenizer) == 256
    got = {0: [], 1: []}
    done = [threading.Event(), threading.Event()]

    def callback(i):
        def cb(token, finished):
            got[i].append(token)
            if finished:
                done[i].set()
        return cb
    long_one, over = [], threading.Event()

    def until_three(token, finished):       # ends its own request after three tokens
        long_one.append((token, finished))
        if len(long_one) == 3:
            engine.abort(long_id[0])
        if finished:
            over.set()
    long_id = [None]
    try:
        for i, p in enumerate(prompts):
            engine.generate_async(p, 6, callback(i))
        assert all(d.wait(120) for d in done)
        long_id[0] = engine.generate_async(prompts[0], 150, until_three)
        assert over.wait(120)
    finally:
        engine.stop()
    assert [got[0], got[1]] == want
    assert long_one[-1] == (-1, True) and 3 <= len(long_one) < 20
    assert [t for t, _ in long_one[:3]] == want[0][:3]
    assert not engine.engine.runner.cache.requests


@pytest.mark.parametrize("dtype,blocks", [("bfloat16", 12), ("float32", 9)])
def test_async_engine_under_threads_aborts_and_preemption(dtype, blocks):
    """Several threads submit requests to one AsyncEngine, end some of them early and wait for
    others, with so few pages that running requests are preempted: every request's callback
    sees exactly one end, nothing is left in the cache, no page is lost."""
    import random
    import threading
    import time
    from lucciola_amd.engine.async_engine import AsyncEngine
    cfg, page, seed = configs.ALL["D"]
    weights = random_weights(cfg, seed, std=0.3)
    engine = engine_for(cfg, weights, page, blocks, dtype, max_tokens_per_step=32, max_seqs=8)
    front = AsyncEngine("", engine=engine)
    problems, ends = [], []

    def worker(wid):
        rng = random.Random(wid)
        waiting = []
        for k in range(12):
            prompt = [rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(1, 60))]
            done, state = threading.Event(), {"tokens": 0, "ends": 0}

            def on_token(tok, finished, state=state, done=done):
                state["tokens"] += 1
                if finished:
                    state["ends"] += 1
                    done.set()
            rid = front.generate_async(prompt, rng.randint(1, 40), on_token,
                                       temperature=rng.choice([0.0, 0.9]), seed=k)
            if rng.random() < 0.3:
                time.sleep(rng.random() * 0.01)
                front.abort(rid)
            waiting.append((done, state))
            if rng.random() < 0.6:
                for d, st in waiting:
                    if not d.wait(120):
                        problems.append(("no end", wid, k))
                ends.extend(st["ends"] for _, st in waiting)
                waiting = []
        for d, st in waiting:
            if not d.wait(120):
                problems.append(("no end", wid))
            ends.append(st["ends"])

    threads = [threading.Thread(target=worker, args=(w,)) for w in range(6)]
    try:
        for th in threads:
            th.start()
        for th in threads:
            th.join()
    finally:
        front.stop()
    assert not problems
    assert len(ends) == 6 * 12 and all(e == 1 for e in ends)
    assert engine.scheduler.num_preemptions > 0
    engine.runner.cache.check()
    assert not engine.runner.cache.requests
    for g in engine.runner.cache.groups:
        assert g.pool.num_free() == blocks


_8B = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 4096,
       "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
       "intermediate_size": 12288, "vocab_size": 151936, "rope_theta": 1000000.0,
       "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 40960,
       "initializer_range": 0.02}


def case_8b():
    if "8b" not in _cache:
        weights = random_weights(_8B, 11, device=DEV)
        prompts = prompts_for(_8B, [150, 37], 12)
        refs = {n: plain_qwen3.forward(_8B, weights, ids) for n, ids in prompts.items()}
        _cache["8b"] = (weights, prompts, refs)
    return _cache["8b"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_the_8b_size(dtype):
    """Two of the 36 layers of the Qwen3-8B-shaped configuration, every size as it is there
    (hidden 4096, 32 query and 8 kv heads of 128, feed-forward 12288, the whole vocabulary of
    151,936 with a head of its own; src/qwen.cc:875-882 is the head): the kernels chosen for
    real sizes (matrix-core products, vector norms, matrix-core attention in bfloat16; FMA
    kernels in float32) against the plain implementation, whole, in portions and token by
    token."""
    weights, prompts, refs = case_8b()
    for family in (traces.whole, lambda p: traces.chunked(p, sizes=(70, 2, 33, 5)),
                   lambda p: traces.tail_decode(p, tail=8)):
        steps = family(prompts)
        runner = make_runner(_8B, weights, 16, traces.max_live_tokens(steps, 16) // 16, dtype, DEV)
        got = replay(runner, steps)
        assert len(got) == 187 and next(iter(got.values())).shape[0] == 151936
        worst = compare(got, _8B, weights, prompts, TOL[dtype], refs)
        print(f"8B-size layers {dtype}: worst relative error {worst:.3e}")
        del runner


def test_8b_size_mixed_steps():
    """Portions of one request beside the decoded tokens of another in ONE step, at the
    8B-shaped layer sizes in bfloat16 (src/qwen.cc:695-728 runs the decode and the prefill
    attention of such a step one after the other): the prefill kernel prepares its own q from
    the raw projections while the decode kernel serves the single tokens, and the products see
    row counts of every kind."""
    weights, prompts, refs = case_8b()
    for seed in (0, 4):
        steps = traces.mixed(prompts, seed=seed, decode_tail=14)
        beside = [len(entries) > 1 and min(len(t) for _, t, _ in entries) == 1
                  and max(len(t) for _, t, _ in entries) > 1 for entries, _ in steps]
        assert any(beside), "no step holds a portion beside a decoded token"
        runner = make_runner(_8B, weights, 16, traces.max_live_tokens(steps, 16) // 16, "bfloat16", DEV)
        got = replay(runner, steps)
        assert len(got) == 187
        worst = compare(got, _8B, weights, prompts, TOL["bfloat16"], refs)
        print(f"8B-size layers, mixed steps (seed {seed}): worst relative error {worst:.3e}")
        del runner


def test_8b_size_requests_that_decode_side_by_side():
    """Six requests at the 8B-shaped sizes whose last tokens are decoded together, six rows a
    step, and twelve: the products of four to sixteen rows, which read large weights in runs
    through LDS, chained through the folded norms as the engine chains them, and the decode
    attention over six and twelve requests at once; against the plain implementation."""
    weights, prompts, refs = case_8b()
    for copies in (3, 6):
        many = {f"{name}{c}": ids for c in range(copies) for name, ids in prompts.items()}
        many_refs = {f"{name}{c}": refs[name] for c in range(copies) for name in prompts}
        tail = 5
        steps = [([(name, list(ids[:-tail]), [len(ids) - tail - 1]) for name, ids in many.items()], [])]
        for i in range(tail, 0, -1):
            steps.append(([(name, [ids[-i]], [0]) for name, ids in many.items()],
                          list(many) if i == 1 else []))
        runner = make_runner(_8B, weights, 16, traces.max_live_tokens(steps, 16) // 16, "bfloat16", DEV,
                             max_seqs=2 * copies)
        got = replay(runner, steps)
        assert len(got) == 2 * copies * (tail + 1)
        worst = compare(got, _8B, weights, many, TOL["bfloat16"], many_refs)
        print(f"8B-size layers, {2 * copies} requests side by side: worst relative error {worst:.3e}")
        del runner


def test_float32_logits_do_not_depend_on_the_cut():
    """In float32 the logits at a position are the same bits however the tokens are cut into
    steps, whatever else is in the batch, whichever pages are used and whatever the page size
    is: every reduction's order is a function of the row alone.  At the 8B-shaped sizes (norm
    rows of 4096, where the kernel's shape once depended on the number of rows) and at tiny C."""
    for cfg, weights, page, lengths in ((_8B, case_8b()[0], 16, [90, 37, 20]),
                                        (configs.TINY_C, random_weights(configs.TINY_C, 2), 16, [70, 33, 50])):
        prompts = prompts_for(cfg, lengths, 77)
        results = []
        for family, pg, shuffle in ((traces.whole, page, False),
                                    (lambda p: traces.chunked(p, sizes=(7, 2, 16, 3, 33)), page, True),
                                    (lambda p: traces.tail_decode(p, tail=6), page, False),
                                    (lambda p: traces.mixed(p, seed=3, decode_tail=4), page, True),
                                    (traces.whole, 4, True)):
            steps = family(prompts)
            blocks = traces.max_live_tokens(steps, 64) // pg + 7
            runner = make_runner(cfg, weights, pg, blocks, "float32", DEV)
            if shuffle:     # other pages, in another order
                import random
                for g in runner.cache.groups:
                    order = list(g.pool._free)
                    random.Random(5).shuffle(order)
                    g.pool._free.clear()
                    g.pool._free.extend(order)
            got = replay(runner, steps)
            results.append({k: v.float() for k, v in got.items()})
            del runner
        for other in results[1:]:
            assert other.keys() == results[0].keys()
            for place, row in results[0].items():
                assert torch.equal(row, other[place]), f"logits at {place} differ between cuts"


def test_cache_sized_from_free_memory():
    """``max_blocks=0`` (the default of the command line and of AsyncEngine): the page count is
    the reference's (src/qwen.cc:527-543: a share of the free memory less 500 MiB over the bytes
    of a page in all layers), capped at what max_seqs requests of the longest context hold."""
    cfg, page, seed = configs.ALL["A"]
    weights = random_weights(cfg, seed, std=0.3)
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), "float32", DEV)
    torch.cuda.synchronize()
    per_page = 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * 4 * page
    for fraction in (2e-6, 0.5):
        free, _ = torch.cuda.mem_get_info(DEV)
        engine = LLMEngine(model, config, EngineConfig(dtype="float32", block_size=page, max_blocks=0,
                                                       memory_fraction=fraction, device=DEV, max_seqs=4,
                                                       max_tokens_per_step=16))
        by_memory = int((free - (500 << 20)) * fraction) // per_page
        cap = 4 * (cfg["max_position_embeddings"] // page)
        assert engine.runner.cache.num_blocks == min(by_memory, cap)
        assert (by_memory < cap) == (fraction < 0.1) and by_memory > 20
        assert engine.runner.cache.storage[0][0][0].shape[0] == engine.runner.cache.num_blocks * engine.runner.cache.groups[0].pieces
        prompts = list(prompts_for(cfg, [5, 11, 17], seed + 30).values())
        got = engine.generate(prompts, SamplingParams(max_new_tokens=8))
        assert got == [plain_qwen3.greedy(cfg, weights, p, 8) for p in prompts]
        del engine


def test_position_table_grows_under_captured_steps():
    """Decode steps replayed from graphs while the rotary table is made anew because a
    position beyond it shows up (a real model's table starts at 16,384 rows; here at 256, so
    that a short run crosses its end twice): logits on both sides of the crossings against
    the plain implementation."""
    from dataclasses import replace
    cfg, page, seed = configs.ALL["D"]
    weights = random_weights(cfg, seed)
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    spec = arch.model_spec(config)
    layers = []
    for layer in spec.layers:
        mixer = layer.parts["mixer"]
        position = mixer.params["position"]
        assert position.params["max_positions"] >= 2048
        layers.append(replace(layer, parts=dict(layer.parts, mixer=mixer.with_params(
            position=position.with_params(max_positions=0, theta=position.params["theta"] + 1)))))
    spec = replace(spec, layers=layers)     # theta + 1: a table of its own, not another test's
    cfg = dict(cfg, rope_theta=cfg["rope_theta"] + 1)
    model = _build(spec, DictSource(weights), "bfloat16", DEV)
    from lucciola_amd.engine.runner import ModelRunner
    runner = ModelRunner(model, EngineConfig(dtype="bfloat16", block_size=page, max_blocks=80,
                                             max_seqs=4, device=DEV))
    prompts = prompts_for(cfg, [600, 530], seed + 3)
    refs = {n: plain_qwen3.forward(cfg, weights, ids) for n, ids in prompts.items()}
    steps = [([(n, ids[:200], []) for n, ids in prompts.items()], [])]
    for i in range(200, 600):
        entries = [(n, [ids[i]], [0]) for n, ids in prompts.items() if i < len(ids)]
        steps.append((entries, []))
    position = model.layers[0].mixer.position
    assert position.capacity() == 0
    got = replay(runner, steps)
    assert position.capacity() >= 600 and position.tables_epoch() >= 3
    assert runner.graph_replays > 300
    compare(got, cfg, weights, prompts, TOL["bfloat16"], refs)


@pytest.mark.parametrize("requests", [20, 40])
def test_many_requests_decode_together(requests):
    """More than 16 requests decode in one step (heads of 128, bfloat16): the products go through
    the tiled kernels, cut along K; the norms sum the shares of the output and down products, the
    attention kernel those of q, k, v; the steps are replayed from graphs.  Every logit row
    against the plain implementation."""
    cfg = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 1024,
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 128,
           "intermediate_size": 1536, "vocab_size": 300, "rope_theta": 100000.0,
           "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 4096,
           "initializer_range": 0.03}
    rng = __import__("random").Random(requests)
    weights = random_weights(cfg, 21)
    prompts = prompts_for(cfg, [rng.randint(2, 40) for _ in range(requests)], 22)
    tail = 5
    steps = []
    names = list(prompts)
    for i in range(0, requests, 8):      # prompts less their last tokens, eight requests a step
        steps.append(([(n, prompts[n][:-tail], []) for n in names[i:i + 8] if len(prompts[n]) > tail], []))
    for k in range(tail):                # then everybody's next token, all in one step
        entries = []
        for n in names:
            ids = prompts[n]
            at = len(ids) - tail + k if len(ids) > tail else k
            if at < len(ids):
                entries.append((n, [ids[at]], [0]))
        steps.append((entries, []))
    steps[-1] = (steps[-1][0], names)
    runner = make_runner(cfg, weights, 16, 4 * requests, "bfloat16", DEV, max_seqs=requests)
    got = replay(runner, steps)
    assert runner.graph_replays >= 2
    assert ops_library().lc_gemm_bf16_shares(requests, (4 + 2 * 2) * 128, 1024) > 1
    compare(got, cfg, weights, prompts, TOL["bfloat16"])


def test_requests_of_uneven_length_decode_through_work_items():
    """One long request among short ones decodes through the planner's list of work items (the
    long request's pages in many shares, the short ones whole), from captured steps; when the
    long one ends, the same number of rows and the same table width go on with lengths of another
    class, which is a captured step of its own.  Every logit row against the plain implementation."""
    cfg = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 512,
           "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 128,
           "intermediate_size": 768, "vocab_size": 300, "rope_theta": 100000.0,
           "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 4096,
           "initializer_range": 0.03}
    weights = peaked(random_weights(cfg, 31))
    lengths = [20, 20, 20, 20, 20, 700]      # (a step of five to eight rows is filled up with copies of its first)
    prompts = prompts_for(cfg, lengths, 32)
    names = list(prompts)
    tail = 6
    steps = [([(n, prompts[n][:-tail], [])], []) for n in names]
    for k in range(tail):
        live = names if k < 3 else names[:-1]         # the long request ends after three steps
        ends = [names[-1]] if k == 2 else (names[:-1] if k == tail - 1 else [])
        steps.append(([(n, [prompts[n][len(prompts[n]) - tail + k]], [0]) for n in live], ends))
    prompts[names[-1]] = prompts[names[-1]][:-3]       # what the plain implementation sees of it
    runner = make_runner(cfg, weights, 16, 80, "bfloat16", DEV, max_seqs=8)
    got = replay(runner, steps)
    lib = ops_library()
    assert lib.lc_attn_decode_by_items(8, 2, 700, 700 + 7 * 20) == 1
    assert lib.lc_attn_decode_by_items(8, 2, 20, 8 * 20) == 0
    assert sorted(runner._graphs) == [(8, 64, ((False, 2),)), (8, 64, ((True, 0),))], list(runner._graphs)
    assert runner.graph_captures == 2 and runner.graph_replays == tail - 2
    compare(got, cfg, weights, prompts, TOL["bfloat16"])


def ops_library():
    from lucciola_amd.kernels import ops
    return ops.library()
