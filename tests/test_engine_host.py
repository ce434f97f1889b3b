"""The engine's host logic on the CPU: the step function, the cache and the batch layout are
run with the plain torch versions of the kernels put in their place, and compared with the
plain whole-sequence implementation.  What these tests cannot see is the kernels themselves
(the ``gpu`` tests cover those)."""
import random

import pytest
import torch

import configs
import plain_qwen3
import reference_ops
import traces
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.engine.batch import StepEntry
from lucciola_amd.engine.loading import random_model
from lucciola_amd.engine.runner import ModelRunner
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.weights.random_init import random_tensors
from lucciola_amd.config.registry import architecture_for


def make(cfg, seed, page, blocks, dtype="float32"):
    arch = architecture_for(cfg)
    spec = arch.model_spec(arch.read_config(cfg))
    weights = dict(random_tensors(declared_tensors(spec), seed, cfg["initializer_range"],
                                  torch.bfloat16))
    from lucciola_amd.engine.loading import _build
    from lucciola_amd.weights.loader import DictSource
    model = _build(spec, DictSource(weights), dtype, "cpu")
    runner = ModelRunner(model, EngineConfig(dtype=dtype, block_size=page, max_blocks=blocks,
                                             max_seqs=4, device="cpu"))
    return runner, weights


def prompts_for(cfg, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(cfg["vocab_size"]) for _ in range(n)]
            for i, n in enumerate(lengths)}


def replay(runner, steps):
    got = {}
    fed = {}
    for entries, end in steps:
        logits = runner.step([StepEntry(n, t, w) for n, t, w in entries])
        row = 0
        for name, tokens, want in entries:
            base = fed.get(name, 0)
            for w in want:
                got[(name, base + w)] = logits[row].double()
                row += 1
            fed[name] = base + len(tokens)
        for name in end:
            runner.finish(name)
            fed.pop(name, None)
        runner.cache.check()
    return got


def compare(got, cfg, weights, prompts, tol):
    worst = 0.0
    for name, ids in prompts.items():
        ref = plain_qwen3.forward(cfg, weights, ids)
        for (n, pos), row in got.items():
            if n != name:
                continue
            err = float((row - ref[pos]).abs().max() / ref[pos].abs().max())
            worst = max(worst, err)
            assert err < tol, f"{name} position {pos}: relative error {err:.3e}"
    return worst


@pytest.mark.parametrize("key", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_step_function_matches_plain(monkeypatch, key, family):
    reference_ops.install(monkeypatch)
    cfg, page, seed = configs.ALL[key]
    lengths = {"A": [5, 11, 17, 40], "B": [1, 9, 30, 64, 45], "C": [70, 33, 50, 3, 61]}[key]
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
