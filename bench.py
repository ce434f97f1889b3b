"""Decode and prefill throughput of the engine on one MI355X, with roofline fractions.

Default run: the layer sizes of the Qwen3-8B-shaped configuration (36 layers, hidden 4096, 32
query heads, 8 kv heads, head size 128, intermediate 12288, vocabulary 151936), random
weights, bfloat16, a batch of 8 requests at a context of 8,192 tokens.  One "step" is one
decode step of the whole batch through the engine's own step function and sampler (greedy).
As in the engine's loop, the sampled tokens reach the next step on the device and the host
reads them while that step runs (`--run-ahead 0`: the host waits for them first).  The cache of the live requests is filled with
random keys and values instead of running their 8,191-token prompts (a decode step's cost
does not depend on what the cache holds); the prefill figure is a real 2,048-token prompt in
one step.  Prints ONE JSON line.  The sections run in this order: the prompt, the other batch
sizes (the largest first), then the headline batch with its own warm-up steps and exactly
``--steps`` timed steps, then the engine's loop and the portions; a GPU that has just been
handed its weights needs a fraction of a second of memory-bound work before its steps take
their settled time, and whichever section runs first pays for it.

Beside the wall-clock time of a step (``ms_per_step``, the headline) the line carries
``gpu_ms`` (the same steps between two HIP events on the stream) and ``host_ms`` (what the host
spends queueing a step, without waiting); ``points`` holds decode at other batch sizes, the
same batch driven through ``LLMEngine`` and its scheduler after real prompts of the context
length (``decode_b8_engine``), and the 2,048-token prompt fed in portions of 576, the
reference's step budget (src/scheduler.cc:48; ``prefill_576``), all in tokens a second.

    python bench.py --gpus 1 --steps 50 --warmup 5
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

SIZES_8B = dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
                rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
                max_position_embeddings=40960, initializer_range=0.02)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--model", default="8b", choices=["8b", "32b", "0.6b"],
                    help="layer sizes: Qwen3-8B-shaped (the default line), 32B- or 0.6B-shaped")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (0: all)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points", default="1,64", help="further decode batch sizes (comma list, '' for none)")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--run-ahead", type=int, default=1, choices=[0, 1],
                    help="1: a step is queued before the host has read the tokens of the one before")
    ap.add_argument("--portion", type=int, default=576,
                    help="also feed the prompt in portions of this many tokens (0: skip)")
    ap.add_argument("--engine-point", type=int, default=1, choices=[0, 1],
                    help="1: also time the batch through LLMEngine and its scheduler, after real prompts")
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed"],
                    help="decode: the default line; mixed: 64 requests with prompts of 16 to 2,048 "
                         "tokens through the scheduler (Qwen3-0.6B-shaped), chunked prefill beside decode")
    ap.add_argument("--new-tokens", type=int, default=128, help="mixed: tokens generated per request")
    ap.add_argument("--max-tokens-per-step", type=int, default=2048, help="mixed: the scheduler's budget")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from lucciola_amd.config.engine_config import EngineConfig
    from lucciola_amd.engine.batch import PENDING, Carry, StepEntry
    from lucciola_amd.engine.loading import random_model
    from lucciola_amd.engine.runner import ModelRunner
    from lucciola_amd.sampling.sampler import Sampler, SamplingParams

    dev = "cuda:0"
    torch.cuda.set_device(0)
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    if args.workload == "mixed":
        return mixed_workload(args, dtype, dev)
    sizes = {"8b": SIZES_8B, "32b": SIZES_32B, "0.6b": SIZES_06B}[args.model]
    layers_full = sizes["num_hidden_layers"]
    args.layers = args.layers or layers_full
    cfg = dict(sizes, architectures=["Qwen3ForCausalLM"], num_hidden_layers=args.layers)
    points = [int(p) for p in args.points.split(",") if p]
    max_batch = max([args.batch] + points)
    steps_total = max(args.steps, 50) + args.warmup + 8
    per_request = args.context + steps_total
    bs = args.block_size
    blocks = max_batch * (-(-per_request // bs)) + (-(-args.prefill_tokens // bs)) + 8

    t0 = time.time()
    model, mcfg = random_model(cfg, seed=0, dtype=dtype, device=dev)
    runner = ModelRunner(model, EngineConfig(dtype=dtype, block_size=bs, max_blocks=blocks,
                                             max_seqs=max_batch + 2, device=dev))
    for ((k, v),) in runner.cache.storage.values():
        k.normal_(0, 0.5)
        v.normal_(0, 0.5)
    sampler = Sampler()
    torch.cuda.synchronize()
    print(f"[bench] model and cache ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)

    L, H, nh, nkv, d = args.layers, mcfg.hidden_size, mcfg.num_attention_heads, mcfg.num_key_value_heads, mcfg.head_dim
    I, V = mcfg.intermediate_size, mcfg.vocab_size
    esize = 2 if args.dtype == "bf16" else 4
    layer_params = (nh + 2 * nkv) * d * H + nh * d * H + 3 * I * H
    weight_bytes = (L * layer_params + V * H) * esize + (2 * L + 1) * H * 4 + 2 * L * d * 4
    kv_bytes_per_token = 2 * L * nkv * d * esize

    def decode_run(batch, steps, warmup):
        """Time ``steps`` decode steps of ``batch`` requests at the context length."""
        names = [f"d{batch}_{i}" for i in range(batch)]
        cache = runner.cache
        for n in names:
            cache.admit(n)
            cache.reserve(n, args.context - 1)
            cache.commit(n)
        gen = torch.Generator().manual_seed(batch)
        tokens = torch.randint(0, V, (batch,), generator=gen).tolist()
        params = [SamplingParams(max_new_tokens=1 << 30)] * batch

        rows = {n: i for i, n in enumerate(names)}
        under_way = None        # the step whose tokens the host has not read yet
        wait = [0.0]            # seconds the host waited for tokens inside the current step

        def one():
            nonlocal tokens, under_way
            if under_way is None:
                logits = runner.step([StepEntry(n, [t], [0]) for n, t in zip(names, tokens)])
            else:
                logits = runner.step([StepEntry(n, [PENDING], [0]) for n in names],
                                     Carry(under_way.ids, rows))
            sampled = sampler.sample_async(logits, params, [0] * batch)
            t_wait = time.perf_counter()
            if under_way is not None:
                tokens = under_way.tokens()
            under_way = sampled
            if not args.run_ahead:
                tokens, under_way = sampled.tokens(), None
            wait[0] += time.perf_counter() - t_wait
        host = 0.0

        def timed():
            nonlocal host
            t_in = time.perf_counter()
            one()
            host += time.perf_counter() - t_in - wait[0]
            wait[0] = 0.0
        for _ in range(warmup):
            one()
        wait[0] = 0.0
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t = time.perf_counter()
        first.record()
        for _ in range(steps):
            timed()
        last.record()
        if under_way is not None:
            tokens = under_way.tokens()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t) * 1e3 / steps
        gpu_ms = first.elapsed_time(last) / steps
        ctx_mid = args.context + warmup + steps / 2.0
        for n in names:
            runner.finish(n)
        bytes_step = weight_bytes + batch * H * esize + batch * ctx_mid * kv_bytes_per_token
        return ms, batch / (ms / 1e3), bytes_step, gpu_ms, host * 1e3 / steps

    def prefill_run(tokens, reps=3):
        gen = torch.Generator().manual_seed(7)
        best = None
        for r in range(reps + 1):
            ids = torch.randint(0, V, (tokens,), generator=gen).tolist()
            torch.cuda.synchronize()
            t = time.perf_counter()
            logits = runner.step([StepEntry(f"p{r}", ids, [tokens - 1])])
            sampler.sample(logits, [SamplingParams()], [0])
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t) * 1e3
            runner.finish(f"p{r}")
            if r > 0:
                best = ms if best is None else min(best, ms)
        flops = 2.0 * tokens * L * layer_params + 2.0 * tokens * tokens * nh * d * L + 2.0 * V * H
        return best, flops

    def prefill_portions(tokens, portion, reps=2):
        """The same prompt fed in portions of ``portion`` tokens, one a step."""
        gen = torch.Generator().manual_seed(9)
        best = None
        for r in range(reps + 1):
            ids = torch.randint(0, V, (tokens,), generator=gen).tolist()
            torch.cuda.synchronize()
            t = time.perf_counter()
            for at in range(0, tokens, portion):
                part = ids[at:at + portion]
                final = at + portion >= tokens
                logits = runner.step([StepEntry(f"q{r}", part, [len(part) - 1] if final else [])])
            sampler.sample(logits, [SamplingParams()], [0])
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t) * 1e3
            runner.finish(f"q{r}")
            if r > 0:
                best = ms if best is None else min(best, ms)
        return best

    def engine_run(batch, steps, warmup):
        """Decode steps of ``batch`` requests driven by LLMEngine and its scheduler: real
        prompts of the context length are fed first (under a budget of 2,048 tokens a step),
        then ``steps`` steps of the engine's loop are timed."""
        from lucciola_amd.engine.llm_engine import LLMEngine
        # requests that are running already decode while the others' prompts are still fed
        new = warmup + steps + 8 + batch * (-(-args.context // 2048) + 1)
        pages = batch * (-(-(args.context + new) // bs)) + 8
        engine = LLMEngine(model, mcfg, EngineConfig(dtype=dtype, block_size=bs, max_blocks=pages,
                                                     max_seqs=batch, max_tokens_per_step=2048, device=dev,
                                                     run_ahead=bool(args.run_ahead)))
        gen = torch.Generator().manual_seed(100 + batch)
        for _ in range(batch):
            engine.add_request(torch.randint(0, V, (args.context - 1,), generator=gen).tolist(),
                               SamplingParams(max_new_tokens=new, ignore_eos=True))
        while engine.scheduler.waiting:
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        t = time.perf_counter()
        got = 0
        for _ in range(steps):
            got += len(engine.step())
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t) * 1e3 / steps
        assert got == steps * batch, f"the engine handed out {got} tokens in {steps} steps of {batch}"
        del engine
        return ms, batch / (ms / 1e3)

    # The prompt and the other batch sizes first, the headline after them: a GPU that has just been handed its weights
    # takes some 0.2 s of memory-bound work to reach its working state (the first twenty steps after the weights are
    # made take 5.55 ms, twenty steps after sixty others 5.40, three hundred in a row 5.42), and serving runs in that state.
    # The headline itself is timed as asked: its own warm-up steps, then exactly --steps steps.
    pms, pflops = prefill_run(args.prefill_tokens)
    print(f"[bench] prefill {args.prefill_tokens}: {pms:.2f} ms", file=sys.stderr, flush=True)
    point_values = {}
    for b in sorted(points, reverse=True):       # the largest first: it has the most steps' worth of time to settle in
        pm, ptps, _, pg, ph = decode_run(b, max(args.steps, 50), 3)
        point_values[f"decode_b{b}"] = round(ptps, 2)
        print(f"[bench] decode batch {b}: {pm:.3f} ms/step (gpu {pg:.3f}, host {ph:.3f})", file=sys.stderr, flush=True)
    ms, tps, bytes_step, gpu_ms, host_ms = decode_run(args.batch, args.steps, args.warmup)
    print(f"[bench] decode batch {args.batch}: {ms:.3f} ms/step (gpu {gpu_ms:.3f}, host {host_ms:.3f})", file=sys.stderr, flush=True)
    achieved = bytes_step / (ms / 1e3) / 1e9
    if args.engine_point:
        em, etps = engine_run(args.batch, max(args.steps, 50), args.warmup)
        point_values[f"decode_b{args.batch}_engine"] = round(etps, 2)
        print(f"[bench] decode batch {args.batch} through the engine's loop: {em:.3f} ms/step", file=sys.stderr, flush=True)
    if args.portion:
        qms = prefill_portions(args.prefill_tokens, args.portion)
        point_values[f"prefill_{args.portion}"] = round(args.prefill_tokens / (qms / 1e3), 1)
        print(f"[bench] prefill {args.prefill_tokens} in portions of {args.portion}: {qms:.2f} ms", file=sys.stderr, flush=True)

    line = {
        "metric": f"decode tok/s (Qwen3-{args.model.upper()}-shaped, batch {args.batch}, context {args.context})",
        "value": round(tps, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "gpu_ms": round(gpu_ms, 4),
        "host_ms": round(host_ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights, random token ids, cache of the live requests filled with random keys/values",
        "config": {"model": f"Qwen3-{args.model.upper()}-shaped", "layers": L, "layers_full": layers_full,
                   "hidden": H, "heads": nh, "kv_heads": nkv, "head_dim": d, "intermediate": I,
                   "vocab": V, "global_batch": args.batch, "seq_len": args.context,
                   "page_size": bs, "prefill_tokens": args.prefill_tokens, "parallelism": "single GPU"},
        "prefill": {"value": round(args.prefill_tokens / (pms / 1e3), 1), "tokens": args.prefill_tokens,
                    "ms": round(pms, 3), "frac": round(pflops / (pms / 1e3) / MFMA_PEAK[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": point_values,
    }
    print(json.dumps(line), flush=True)
    return 0


SIZES_32B = dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64,
                 num_key_value_heads=8, head_dim=128, intermediate_size=25600, vocab_size=151936,
                 rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
                 max_position_embeddings=40960, initializer_range=0.02)

SIZES_06B = dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16,
                 num_key_value_heads=8, head_dim=128, intermediate_size=3072, vocab_size=151936,
                 rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
                 max_position_embeddings=40960, initializer_range=0.02)


def mixed_workload(args, dtype, dev) -> int:
    """64 requests with random prompts of 16 to 2,048 tokens, all submitted at once; the
    scheduler cuts the prompts into portions under its token budget beside the decode tokens of
    the requests that are already running."""
    import random
    import torch
    from lucciola_amd.config.engine_config import EngineConfig
    from lucciola_amd.engine.llm_engine import LLMEngine
    from lucciola_amd.sampling.sampler import SamplingParams

    cfg = dict(SIZES_06B, architectures=["Qwen3ForCausalLM"])
    rng = random.Random(0)
    prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(16, 2048))] for _ in range(64)]
    total_tokens = sum(len(p) for p in prompts) + 64 * args.new_tokens
    blocks = -(-total_tokens // args.block_size) + 64
    engine = LLMEngine.from_random(cfg, 0, EngineConfig(
        dtype=dtype, block_size=args.block_size, max_blocks=blocks, max_seqs=64,
        max_tokens_per_step=args.max_tokens_per_step, device=dev, run_ahead=bool(args.run_ahead)))
    params = SamplingParams(max_new_tokens=args.new_tokens, ignore_eos=True)
    engine.generate(prompts[:4], SamplingParams(max_new_tokens=4, ignore_eos=True))   # warm-up
    torch.cuda.synchronize()
    steps0 = engine.runner.steps
    t = time.perf_counter()
    outputs = engine.generate(prompts, params)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t
    generated = sum(len(o) for o in outputs)
    prompt_tokens = sum(len(p) for p in prompts)
    line = {
        "metric": "tokens/s, 64 requests with prompts of 16..2048 tokens (Qwen3-0.6B-shaped), chunked prefill beside decode",
        "value": round((prompt_tokens + generated) / seconds, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": engine.runner.steps - steps0, "warmup": 1,
        "ms_per_step": round(seconds * 1e3 / max(1, engine.runner.steps - steps0), 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights, random token ids",
        "config": {"model": "Qwen3-0.6B-shaped", "layers": cfg["num_hidden_layers"], "requests": 64,
                   "prompt_tokens": prompt_tokens, "generated_tokens": generated,
                   "max_tokens_per_step": args.max_tokens_per_step, "page_size": args.block_size,
                   "preemptions": engine.scheduler.num_preemptions, "seconds": round(seconds, 3),
                   "generated_tokens_per_s": round(generated / seconds, 1)},
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
