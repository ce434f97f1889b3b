"""Decode and prefill throughput of the engine on one MI355X, with roofline fractions.

Default run: the layer sizes of the Qwen3-8B-shaped configuration (36 layers, hidden 4096, 32
query heads, 8 kv heads, head size 128, intermediate 12288, vocabulary 151936), random
weights, bfloat16, a batch of 8 requests at a context of 8,192 tokens.  One "step" is one
decode step of the whole batch through the engine's own step function and sampler (greedy).
As in the engine's loop, the sampled tokens reach the next step on the device and the host
reads them while that step runs (`--run-ahead 0`: the host waits for them first).  The cache of
the live requests is filled with random keys and values instead of running their prompts (a
decode step's cost does not depend on what the cache holds); the prefill figure is a real
2,048-token prompt in one step.  Prints ONE JSON line.

The sections run in this order: the prompt, the other decode points of this model (the largest
batch first), then the headline batch with its own warm-up steps and exactly ``--steps`` timed
steps, then the engine's loop and the portions; then, unless ``--others 0``, the other two
shapes whose runs the baseline names: Qwen3-32B-shaped (decode at batch 1 and 32 at a context
of 8,192, a 2,048-token prompt) and the Qwen3-0.6B-shaped mixed workload (64 requests with
prompts of 16 to 2,048 tokens through the scheduler, portions beside decoding).  A GPU that has
just been handed its weights needs a fraction of a second of memory-bound work before its
steps take their settled time, and whichever section runs first pays for it.

Beside the wall-clock time of a step (``ms_per_step``, the headline) the line carries
``gpu_ms`` (the same steps between two HIP events on the stream) and ``host_ms`` (what the host
spends on a step without waiting: the runner's own account of reserving pages, laying out the
batch and launching, plus queueing the sampler; ``host_split_ms`` has the parts, and the same
for the engine's loop from ``LLMEngine.stats()``).  ``points`` holds, in tokens a second:
decode at the other batch sizes at the headline's context (``decode_b1``, ``decode_b64``) and
at a context of 1,024 tokens (``decode_b1_ctx1024``, ...: the length of the prompts that the
baseline's runs decode after; there also a batch of 256, ``decode_b256_ctx1024``), a batch of 64
requests of uneven length (one at the headline's context among 63 of 512 tokens:
``decode_b64_one_long``), the headline's batch driven through ``LLMEngine`` and its scheduler
after real prompts of the context length (``decode_b8_engine``), the 2,048-token prompt fed in
portions of 576, the reference's step budget (src/scheduler.cc:48; ``prefill_576``), and the
other shapes (``32b_decode_b1``, ``32b_decode_b32``, ``32b_prefill_2048``, ``0.6b_mixed``).
``fractions`` gives each point's share of its roofline: for decode the bytes a step has to
read (every weight once, the cache of the live requests) over its time over 8 TB/s; for
prompts, and for the mixed workload, the model's flops over the time over 2.5 PFLOP/s.

    python bench.py --gpus 1 --steps 50 --warmup 5
"""
import argparse
import gc
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

SIZES_32B = dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64,
                 num_key_value_heads=8, head_dim=128, intermediate_size=25600, vocab_size=151936,
                 rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
                 max_position_embeddings=40960, initializer_range=0.02)

SIZES_06B = dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16,
                 num_key_value_heads=8, head_dim=128, intermediate_size=3072, vocab_size=151936,
                 rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
                 max_position_embeddings=40960, initializer_range=0.02)


SIZES_17B = dict(num_hidden_layers=28, hidden_size=2048, num_attention_heads=16,
                 num_key_value_heads=8, head_dim=128, intermediate_size=6144, vocab_size=151936,
                 rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
                 max_position_embeddings=40960, initializer_range=0.02)

SIZES_4B = dict(num_hidden_layers=36, hidden_size=2560, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, intermediate_size=9728, vocab_size=151936,
                rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
                max_position_embeddings=40960, initializer_range=0.02)

SIZES_14B = dict(num_hidden_layers=40, hidden_size=5120, num_attention_heads=40,
                 num_key_value_heads=8, head_dim=128, intermediate_size=17408, vocab_size=151936,
                 rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
                 max_position_embeddings=40960, initializer_range=0.02)

SIZES = {"8b": SIZES_8B, "32b": SIZES_32B, "0.6b": SIZES_06B, "1.7b": SIZES_17B, "4b": SIZES_4B, "14b": SIZES_14B}


def say(text):
    print(f"[bench] {text}", file=sys.stderr, flush=True)


class ModelBench:
    """One model with random weights and a cache for its largest run, and the timed runs."""

    def __init__(self, sizes, layers, dtype, dev, block_size, max_batch, max_context, prefill_tokens,
                 run_ahead, spare_steps, max_seqs=0):
        import torch
        from lucciola_amd.config.engine_config import EngineConfig
        from lucciola_amd.engine.loading import random_model
        from lucciola_amd.engine.runner import ModelRunner
        from lucciola_amd.sampling.sampler import Sampler

        self.torch, self.dev, self.bs, self.run_ahead = torch, dev, block_size, run_ahead
        self.dtype = "bfloat16" if dtype == "bf16" else "float32"
        self.dtype_key = dtype
        self.layers_full = sizes["num_hidden_layers"]
        self.L = layers or self.layers_full
        cfg = dict(sizes, architectures=["Qwen3ForCausalLM"], num_hidden_layers=self.L)
        per_request = max_context + spare_steps
        blocks = max_batch * (-(-per_request // block_size)) + (-(-prefill_tokens // block_size)) + 8
        t0 = time.time()
        self.model, self.mcfg = random_model(cfg, seed=0, dtype=self.dtype, device=dev)
        self.runner = ModelRunner(self.model, EngineConfig(dtype=self.dtype, block_size=block_size,
                                                           max_blocks=blocks, max_seqs=max(max_batch, max_seqs) + 2, device=dev))
        for ((k, v),) in self.runner.cache.storage.values():
            k.normal_(0, 0.5)
            v.normal_(0, 0.5)
        self.sampler = Sampler()
        torch.cuda.synchronize()
        say(f"{self.L} layers of width {self.mcfg.hidden_size} and a cache of {blocks} pages ready in "
            f"{time.time() - t0:.1f} s")
        m = self.mcfg
        self.H, self.nh, self.nkv, self.d = m.hidden_size, m.num_attention_heads, m.num_key_value_heads, m.head_dim
        self.I, self.V = m.intermediate_size, m.vocab_size
        self.esize = 2 if dtype == "bf16" else 4
        self.layer_params = (self.nh + 2 * self.nkv) * self.d * self.H + self.nh * self.d * self.H + 3 * self.I * self.H
        self.weight_bytes = ((self.L * self.layer_params + self.V * self.H) * self.esize
                             + (2 * self.L + 1) * self.H * 4 + 2 * self.L * self.d * 4)
        self.kv_bytes_per_token = 2 * self.L * self.nkv * self.d * self.esize

    def close(self):
        self.runner = self.model = self.sampler = None
        gc.collect()
        self.torch.cuda.empty_cache()

    def decode_run(self, batch, context, steps, warmup):
        """Time ``steps`` decode steps of ``batch`` requests that hold ``context`` tokens each (a
        list: one length a request).  Returns a dict: ms, tokens a second, the bytes a step must
        read, gpu ms, host ms and its parts."""
        from lucciola_amd.engine.batch import PENDING, Carry, StepEntry
        from lucciola_amd.sampling.sampler import SamplingParams
        torch, runner, sampler = self.torch, self.runner, self.sampler
        contexts = list(context) if isinstance(context, (list, tuple)) else [context] * batch
        assert len(contexts) == batch
        names = [f"d{batch}_{contexts[0]}_{contexts[-1]}_{i}" for i in range(batch)]
        cache = runner.cache
        for n, c in zip(names, contexts):
            cache.admit(n)
            cache.reserve(n, c - 1)
            cache.commit(n)
        gen = torch.Generator().manual_seed(batch)
        tokens = torch.randint(0, self.V, (batch,), generator=gen).tolist()
        params = [SamplingParams(max_new_tokens=1 << 30)] * batch
        rows = {n: i for i, n in enumerate(names)}
        state = {"under_way": None, "tokens": tokens, "sample_s": 0.0}

        def one():
            under_way = state["under_way"]
            if under_way is None:
                logits = runner.step([StepEntry(n, [t], [0]) for n, t in zip(names, state["tokens"])])
            else:
                logits = runner.step([StepEntry(n, [PENDING], [0]) for n in names], Carry(under_way.ids, rows))
            t_in = time.perf_counter()
            sampled = sampler.sample_async(logits, params, [0] * batch)
            state["sample_s"] += time.perf_counter() - t_in
            if under_way is not None:
                state["tokens"] = under_way.tokens()
            state["under_way"] = sampled
            if not self.run_ahead:
                state["tokens"], state["under_way"] = sampled.tokens(), None

        for _ in range(warmup):
            one()
        state["sample_s"] = 0.0
        before = dict(runner.times)
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t = time.perf_counter()
        first.record()
        for _ in range(steps):
            one()
        last.record()
        if state["under_way"] is not None:
            state["under_way"].tokens()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t) * 1e3 / steps
        gpu_ms = first.elapsed_time(last) / steps
        split = {k: (runner.times[k] - before[k]) * 1e3 / steps for k in before}
        split["sample"] = state["sample_s"] * 1e3 / steps
        ctx_mid = sum(contexts) / batch + warmup + steps / 2.0
        for n in names:
            runner.finish(n)
        bytes_step = self.weight_bytes + batch * self.H * self.esize + batch * ctx_mid * self.kv_bytes_per_token
        return {"ms": ms, "tps": batch / (ms / 1e3), "bytes": bytes_step, "gpu_ms": gpu_ms,
                "host_ms": sum(split.values()), "split": split,
                "frac": bytes_step / (ms / 1e3) / 1e9 / HBM_PEAK_GBS}

    def prefill_flops(self, tokens):
        return (2.0 * tokens * self.L * self.layer_params + 2.0 * tokens * tokens * self.nh * self.d * self.L
                + 2.0 * self.V * self.H)

    def prefill_run(self, tokens, reps=3):
        from lucciola_amd.engine.batch import StepEntry
        from lucciola_amd.sampling.sampler import SamplingParams
        torch = self.torch
        gen = torch.Generator().manual_seed(7)
        best = None
        for r in range(reps + 1):
            ids = torch.randint(0, self.V, (tokens,), generator=gen).tolist()
            torch.cuda.synchronize()
            t = time.perf_counter()
            logits = self.runner.step([StepEntry(f"p{r}", ids, [tokens - 1])])
            self.sampler.sample(logits, [SamplingParams()], [0])
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t) * 1e3
            self.runner.finish(f"p{r}")
            if r > 0:
                best = ms if best is None else min(best, ms)
        return best, self.prefill_flops(tokens)

    def prefill_portions(self, tokens, portion, reps=2):
        """The same prompt fed in portions of ``portion`` tokens, one a step."""
        from lucciola_amd.engine.batch import StepEntry
        from lucciola_amd.sampling.sampler import SamplingParams
        torch = self.torch
        gen = torch.Generator().manual_seed(9)
        best = None
        for r in range(reps + 1):
            ids = torch.randint(0, self.V, (tokens,), generator=gen).tolist()
            torch.cuda.synchronize()
            t = time.perf_counter()
            for at in range(0, tokens, portion):
                part = ids[at:at + portion]
                final = at + portion >= tokens
                logits = self.runner.step([StepEntry(f"q{r}", part, [len(part) - 1] if final else [])])
            self.sampler.sample(logits, [SamplingParams()], [0])
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t) * 1e3
            self.runner.finish(f"q{r}")
            if r > 0:
                best = ms if best is None else min(best, ms)
        return best

    def engine_run(self, batch, context, steps, warmup):
        """Decode steps of ``batch`` requests driven by LLMEngine and its scheduler: real
        prompts of the context length are fed first (under a budget of 2,048 tokens a step),
        then ``steps`` steps of the engine's loop are timed.  Returns ms a step, tokens a
        second and the host's time by where it went, from ``LLMEngine.stats()``."""
        from lucciola_amd.config.engine_config import EngineConfig
        from lucciola_amd.engine.llm_engine import LLMEngine
        from lucciola_amd.sampling.sampler import SamplingParams
        torch = self.torch
        # requests that are running already decode while the others' prompts are still fed
        new = warmup + steps + 8 + batch * (-(-context // 2048) + 1)
        pages = batch * (-(-(context + new) // self.bs)) + 8
        engine = LLMEngine(self.model, self.mcfg, EngineConfig(
            dtype=self.dtype, block_size=self.bs, max_blocks=pages, max_seqs=batch,
            max_tokens_per_step=2048, device=self.dev, run_ahead=bool(self.run_ahead)))
        gen = torch.Generator().manual_seed(100 + batch)
        for _ in range(batch):
            engine.add_request(torch.randint(0, self.V, (context - 1,), generator=gen).tolist(),
                               SamplingParams(max_new_tokens=new, ignore_eos=True))
        while engine.scheduler.waiting:
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        before = engine.stats()
        t = time.perf_counter()
        got = 0
        for _ in range(steps):
            got += len(engine.step())
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t) * 1e3 / steps
        after = engine.stats()
        assert got == steps * batch, f"the engine handed out {got} tokens in {steps} steps of {batch}"
        split = {k[:-2]: (after[k] - before[k]) * 1e3 / steps
                 for k in ("schedule_s", "reserve_s", "batch_s", "launch_s", "sample_s", "wait_s")}
        del engine
        return ms, batch / (ms / 1e3), split


def mixed_workload(dtype, dev, block_size, run_ahead, new_tokens, max_tokens_per_step):
    """64 requests with random prompts of 16 to 2,048 tokens, all submitted at once; the
    scheduler cuts the prompts into portions under its token budget beside the decode tokens of
    the requests that are already running (Qwen3-0.6B-shaped).  Returns the figures of the run."""
    import random
    import torch
    from lucciola_amd.config.engine_config import EngineConfig
    from lucciola_amd.engine.llm_engine import LLMEngine
    from lucciola_amd.sampling.sampler import SamplingParams

    cfg = dict(SIZES_06B, architectures=["Qwen3ForCausalLM"])
    rng = random.Random(0)
    prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(16, 2048))] for _ in range(64)]
    total_tokens = sum(len(p) for p in prompts) + 64 * new_tokens
    blocks = -(-total_tokens // block_size) + 64
    engine = LLMEngine.from_random(cfg, 0, EngineConfig(
        dtype="bfloat16" if dtype == "bf16" else "float32", block_size=block_size, max_blocks=blocks,
        max_seqs=64, max_tokens_per_step=max_tokens_per_step, device=dev, run_ahead=bool(run_ahead)))
    params = SamplingParams(max_new_tokens=new_tokens, ignore_eos=True)
    engine.generate(prompts[:4], SamplingParams(max_new_tokens=4, ignore_eos=True))   # warm-up
    torch.cuda.synchronize()
    steps0 = engine.runner.steps
    t = time.perf_counter()
    outputs = engine.generate(prompts, params)
    torch.cuda.synchronize()
    seconds = time.perf_counter() - t
    generated = sum(len(o) for o in outputs)
    prompt_tokens = sum(len(p) for p in prompts)
    # the model's flops for this work: every token through every layer's products and the
    # attention over what precedes it, the head for every sampled token
    c = cfg
    L, H, nh, nkv, d, I, V = (c["num_hidden_layers"], c["hidden_size"], c["num_attention_heads"],
                              c["num_key_value_heads"], c["head_dim"], c["intermediate_size"], c["vocab_size"])
    layer_params = (nh + 2 * nkv) * d * H + nh * d * H + 3 * I * H
    flops = 0.0
    for p in prompts:
        n = len(p) + new_tokens
        flops += 2.0 * n * L * layer_params + 2.0 * n * n * nh * d * L + 2.0 * new_tokens * V * H
    steps = engine.runner.steps - steps0
    out = {"tps": (prompt_tokens + generated) / seconds, "seconds": seconds, "steps": steps,
           "prompt_tokens": prompt_tokens, "generated": generated,
           "preemptions": engine.scheduler.num_preemptions,
           "frac": flops / seconds / MFMA_PEAK[dtype]}
    del engine
    gc.collect()
    torch.cuda.empty_cache()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=8192)
    ap.add_argument("--model", default="8b", choices=sorted(SIZES),
                    help="layer sizes: Qwen3-8B-shaped (the default line), or another size of the family")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (0: all)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points", default="1,64", help="further decode batch sizes (comma list, '' for none)")
    ap.add_argument("--short-points", default="256",
                    help="further batch sizes measured at the short context only (those that fit the cache)")
    ap.add_argument("--short-context", type=int, default=1024,
                    help="also decode at this context, at the headline's batch and the batches of --points (0: skip)")
    ap.add_argument("--uneven-point", type=int, default=1, choices=[0, 1],
                    help="1: also decode a batch of 64 with one request at the full context among 63 of 512 tokens")
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--run-ahead", type=int, default=1, choices=[0, 1],
                    help="1: a step is queued before the host has read the tokens of the one before")
    ap.add_argument("--portion", type=int, default=576,
                    help="also feed the prompt in portions of this many tokens (0: skip)")
    ap.add_argument("--engine-point", type=int, default=1, choices=[0, 1],
                    help="1: also time the batch through LLMEngine and its scheduler, after real prompts")
    ap.add_argument("--others", type=int, default=-1, choices=[-1, 0, 1],
                    help="1: also run the 32B-shaped points and the 0.6B-shaped mixed workload; "
                         "-1 (default): only in the default run (8B-shaped, bf16, all layers)")
    ap.add_argument("--workload", default="decode", choices=["decode", "mixed"],
                    help="decode: the default line; mixed: only the 0.6B-shaped mixed workload, as a line of its own")
    ap.add_argument("--new-tokens", type=int, default=128, help="mixed: tokens generated per request")
    ap.add_argument("--max-tokens-per-step", type=int, default=2048, help="mixed: the scheduler's budget")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.workload == "mixed":
        m = mixed_workload(args.dtype, dev, args.block_size, args.run_ahead, args.new_tokens, args.max_tokens_per_step)
        line = {
            "metric": "tokens/s, 64 requests with prompts of 16..2048 tokens (Qwen3-0.6B-shaped), chunked prefill beside decode",
            "value": round(m["tps"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": m["steps"], "warmup": 1,
            "ms_per_step": round(m["seconds"] * 1e3 / max(1, m["steps"]), 3),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
            "data": "synthetic: random weights, random token ids",
            "config": {"model": "Qwen3-0.6B-shaped", "layers": SIZES_06B["num_hidden_layers"], "requests": 64,
                       "prompt_tokens": m["prompt_tokens"], "generated_tokens": m["generated"],
                       "max_tokens_per_step": args.max_tokens_per_step, "page_size": args.block_size,
                       "preemptions": m["preemptions"], "seconds": round(m["seconds"], 3),
                       "generated_tokens_per_s": round(m["generated"] / m["seconds"], 1)},
        }
        print(json.dumps(line), flush=True)
        return 0

    sizes = SIZES[args.model]
    points = [int(p) for p in args.points.split(",") if p]
    others = args.others == 1 or (args.others == -1 and args.model == "8b" and not args.layers
                                  and args.dtype == "bf16")
    point_steps = max(args.steps, 50)
    short_points = [int(p) for p in args.short_points.split(",") if p] if args.short_context else []
    most = max([args.batch] + points)
    # the larger batches of the short context must fit the cache that the longest run needs
    short_points = [b for b in short_points
                    if b * (args.short_context + point_steps + 16) <= most * max(args.context, args.short_context)]
    bench = ModelBench(sizes, args.layers, args.dtype, dev, args.block_size, most,
                       max(args.context, args.short_context), args.prefill_tokens, args.run_ahead,
                       spare_steps=point_steps + args.warmup + 8, max_seqs=max([0] + short_points))
    values, fractions = {}, {}

    # The prompt and the other decode points first, the headline after them: a GPU that has just been handed its weights
    # takes some 0.2 s of memory-bound work to reach its working state (the first twenty steps after the weights are
    # made take 5.55 ms, twenty steps after sixty others 5.40, three hundred in a row 5.42), and serving runs in that state.
    # The headline itself is timed as asked: its own warm-up steps, then exactly --steps steps.
    pms, pflops = bench.prefill_run(args.prefill_tokens)
    say(f"prefill {args.prefill_tokens}: {pms:.2f} ms")
    for b in sorted(points, reverse=True):       # the largest first: it has the most steps' worth of time to settle in
        r = bench.decode_run(b, args.context, point_steps, 3)
        values[f"decode_b{b}"], fractions[f"decode_b{b}"] = round(r["tps"], 2), round(r["frac"], 4)
        say(f"decode batch {b}: {r['ms']:.3f} ms/step (gpu {r['gpu_ms']:.3f}, host {r['host_ms']:.3f}), "
            f"{r['frac']:.3f} of the HBM peak")
    if args.short_context and args.short_context != args.context:
        for b in sorted(set(points + [args.batch] + short_points), reverse=True):
            r = bench.decode_run(b, args.short_context, point_steps, 3)
            key = f"decode_b{b}_ctx{args.short_context}"
            values[key], fractions[key] = round(r["tps"], 2), round(r["frac"], 4)
            say(f"decode batch {b} at context {args.short_context}: {r['ms']:.3f} ms/step, {r['frac']:.3f} of the HBM peak")
    if args.uneven_point and 64 in points and args.context >= 8192:
        # requests of uneven length, as a serving batch has them: one long request among 63 short ones
        r = bench.decode_run(64, [args.context] + [512] * 63, point_steps, 3)
        values["decode_b64_one_long"], fractions["decode_b64_one_long"] = round(r["tps"], 2), round(r["frac"], 4)
        say(f"decode batch 64, one request of {args.context} tokens among 63 of 512: {r['ms']:.3f} ms/step, "
            f"{r['frac']:.3f} of the HBM peak")
    head = bench.decode_run(args.batch, args.context, args.steps, args.warmup)
    ms, tps = head["ms"], head["tps"]
    say(f"decode batch {args.batch}: {ms:.3f} ms/step (gpu {head['gpu_ms']:.3f}, host {head['host_ms']:.3f})")
    achieved = head["bytes"] / (ms / 1e3) / 1e9
    host_split = {"step": {k: round(v, 4) for k, v in head["split"].items()}}
    if args.engine_point:
        em, etps, esplit = bench.engine_run(args.batch, args.context, point_steps, args.warmup)
        values[f"decode_b{args.batch}_engine"] = round(etps, 2)
        fractions[f"decode_b{args.batch}_engine"] = round(head["bytes"] / (em / 1e3) / 1e9 / HBM_PEAK_GBS, 4)
        host_split["engine"] = {k: round(v, 4) for k, v in esplit.items()}
        say(f"decode batch {args.batch} through the engine's loop: {em:.3f} ms/step")
    if args.portion:
        qms = bench.prefill_portions(args.prefill_tokens, args.portion)
        values[f"prefill_{args.portion}"] = round(args.prefill_tokens / (qms / 1e3), 1)
        fractions[f"prefill_{args.portion}"] = round(pflops / (qms / 1e3) / MFMA_PEAK[args.dtype], 4)
        say(f"prefill {args.prefill_tokens} in portions of {args.portion}: {qms:.2f} ms")
    L, H, nh, nkv, d, I, V = bench.L, bench.H, bench.nh, bench.nkv, bench.d, bench.I, bench.V
    layers_full = bench.layers_full
    bench.close()

    if others:
        big = ModelBench(SIZES_32B, 0, args.dtype, dev, args.block_size, 32, args.context, args.prefill_tokens,
                         args.run_ahead, spare_steps=point_steps + 16)
        bms, bflops = big.prefill_run(args.prefill_tokens, reps=2)
        values["32b_prefill_2048"] = round(args.prefill_tokens / (bms / 1e3), 1)
        fractions["32b_prefill_2048"] = round(bflops / (bms / 1e3) / MFMA_PEAK[args.dtype], 4)
        say(f"32B-shaped prefill {args.prefill_tokens}: {bms:.2f} ms")
        for b in (32, 1):
            r = big.decode_run(b, args.context, point_steps, 3)
            values[f"32b_decode_b{b}"], fractions[f"32b_decode_b{b}"] = round(r["tps"], 2), round(r["frac"], 4)
            say(f"32B-shaped decode batch {b}: {r['ms']:.3f} ms/step, {r['frac']:.3f} of the HBM peak")
        big.close()
        m = mixed_workload(args.dtype, dev, args.block_size, args.run_ahead, args.new_tokens, args.max_tokens_per_step)
        values["0.6b_mixed"], fractions["0.6b_mixed"] = round(m["tps"], 1), round(m["frac"], 4)
        say(f"0.6B-shaped mixed workload: {m['tps']:.0f} tokens/s in {m['seconds']:.2f} s, {m['steps']} steps")

    line = {
        "metric": f"decode tok/s (Qwen3-{args.model.upper()}-shaped, batch {args.batch}, context {args.context})",
        "value": round(tps, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "gpu_ms": round(head["gpu_ms"], 4),
        "host_ms": round(head["host_ms"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights, random token ids, cache of the live requests filled with random keys/values",
        "config": {"model": f"Qwen3-{args.model.upper()}-shaped", "layers": L, "layers_full": layers_full,
                   "hidden": H, "heads": nh, "kv_heads": nkv, "head_dim": d, "intermediate": I,
                   "vocab": V, "global_batch": args.batch, "seq_len": args.context,
                   "page_size": args.block_size, "prefill_tokens": args.prefill_tokens, "parallelism": "single GPU"},
        "prefill": {"value": round(args.prefill_tokens / (pms / 1e3), 1), "tokens": args.prefill_tokens,
                    "ms": round(pms, 3), "frac": round(pflops / (pms / 1e3) / MFMA_PEAK[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "points": values,
        "fractions": fractions,
        "host_split_ms": host_split,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
