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
