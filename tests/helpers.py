"""Shared by the CPU and GPU tests: building a tiny model with random weights, replaying a
trace through the runner, comparing with the plain implementation."""
import random

import torch

import plain_qwen3
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.engine.batch import StepEntry
from lucciola_amd.engine.loading import _build
from lucciola_amd.engine.runner import ModelRunner
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.weights.loader import DictSource
from lucciola_amd.weights.random_init import random_tensors


def random_weights(cfg, seed, std=None, dtype=torch.bfloat16, device="cpu"):
    """The random weights of (cfg, seed); made on ``device`` (the values are the same on every
    device), returned on the CPU."""
    arch = architecture_for(cfg)
    spec = arch.model_spec(arch.read_config(cfg))
    return {name: t.cpu() for name, t in random_tensors(
        declared_tensors(spec), seed, cfg["initializer_range"] if std is None else std, dtype,
        device=device)}


def make_runner(cfg, weights, page, blocks, dtype, device, max_seqs=4):
    arch = architecture_for(cfg)
    spec = arch.model_spec(arch.read_config(cfg))
    model = _build(spec, DictSource(weights), dtype, device)
    return ModelRunner(model, EngineConfig(dtype=dtype, block_size=page, max_blocks=blocks,
                                           max_seqs=max_seqs, device=device))


def prompts_for(cfg, lengths, seed):
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(cfg["vocab_size"]) for _ in range(n)]
            for i, n in enumerate(lengths)}


def replay(runner, steps, check=True):
    """Run a trace; returns {(request, position): logits row (float64, CPU)}."""
    got, fed = {}, {}
    for entries, end in steps:
        logits = runner.step([StepEntry(n, t, w) for n, t, w in entries]).double().cpu()
        row = 0
        for name, tokens, want in entries:
            base = fed.get(name, 0)
            for w in want:
                got[(name, base + w)] = logits[row]
                row += 1
            fed[name] = base + len(tokens)
        for name in end:
            runner.finish(name)
            fed.pop(name, None)
        if check:
            runner.cache.check()
    return got


def compare(got, cfg, weights, prompts, tol, refs=None):
    """Every row of ``got`` against the plain whole-sequence logits; the error of a row is
    max |difference| / max |logit|.  Returns the worst row's error."""
    worst, first_bad = 0.0, None
    for name, ids in prompts.items():
        ref = refs[name] if refs is not None else plain_qwen3.forward(cfg, weights, ids)
        for pos in range(len(ids)):
            if (name, pos) not in got:
                continue
            row = got[(name, pos)]
            assert torch.isfinite(row).all(), f"{name} position {pos}: logits are not finite"
            err = float((row - ref[pos]).abs().max() / ref[pos].abs().max())
            if err > worst:
                worst = err
            if err >= tol and first_bad is None:
                first_bad = (name, pos, err)
    assert first_bad is None, (f"first wrong place: request {first_bad[0]} position {first_bad[1]} "
                               f"relative error {first_bad[2]:.3e} (tolerance {tol:.1e}, worst {worst:.3e})")
    return worst
