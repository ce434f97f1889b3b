"""The command line, in the manner of the reference's ``lucciola_chat``
(examples/qwen_dynamic.cc:40-106: load the model, make the paged cache with ``max_blocks`` pages
of ``block_size`` tokens, read a request per input line until ``exit``, run the scheduler loop
and stream what is generated, at most 100 tokens a request).

Requests are token ids: a line of ids separated by blanks or commas.  Where the model folder
holds a ``vocab.json``, ``--prompt`` and ``--text`` take text as the reference does: encoded by
longest match against the vocabulary (src/tokenizer.cc:87-132) inside the reference's chat
format (examples/qwen_dynamic.cc:48-66), and what is generated is printed as text.  Options
carry the reference's names where it has them: ``--max-blocks`` and ``--block-size`` are the
arguments of ``AsyncEngine(model_path, max_blocks, block_size)`` (include/async_engine.h:24-25),
``--max-new-tokens`` that of ``generate_async``.

    python -m lucciola_amd --model DIR                       # ids from standard input
    python -m lucciola_amd --model DIR --prompt-ids 1,2,3 --prompt-ids 4,5
    python -m lucciola_amd --model DIR --text                # a line of text per request
    python -m lucciola_amd --model DIR --prompt "Why is the sky blue?"
    python -m lucciola_amd --random-config config.json --seed 0 --write-model DIR
"""
from __future__ import annotations

import argparse
import json
import re
import sys
from typing import List


def _ids(text: str) -> List[int]:
    return [int(t) for t in re.split(r"[,\s]+", text.strip()) if t]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="lucciola_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--max-blocks", "--num-pages", dest="max_blocks", type=int, default=0,
                    help="pages of the cache; 0 sizes it from free memory (the reference's default)")
    ap.add_argument("--block-size", "--page-size", dest="block_size", type=int, default=16,
                    help="tokens in a page (multiples of 16 are served by the matrix-core attention kernels)")
    ap.add_argument("--mem-fraction", type=float, default=0.90,
                    help="with --max-blocks 0: share of the free memory the cache may take "
                         "(the reference's 0.90, src/async_engine.cc:13)")
    ap.add_argument("--max-new-tokens", type=int, default=100)
    ap.add_argument("--temperature", type=float, default=0.0, help="0 is greedy")
    ap.add_argument("--seed", "--sample-seed", dest="seed", type=int, default=0,
                    help="of the sampler, or of --random-config")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32", "bf16", "fp32"])
    ap.add_argument("--max-tokens-per-step", type=int, default=2048)
    ap.add_argument("--max-seqs", type=int, default=256)
    ap.add_argument("--ignore-eos", action="store_true")
    ap.add_argument("--prompt-ids", action="append", default=[],
                    help="a request as comma-separated token ids (may be given several times)")
    ap.add_argument("--prompt", action="append", default=[],
                    help="a request as text (needs vocab.json in the model folder; may be given several times)")
    ap.add_argument("--text", action="store_true",
                    help="lines of standard input are text, not token ids (needs vocab.json)")
    ap.add_argument("--no-chat-format", action="store_true",
                    help="encode text as it is, without the reference's chat format around it")
    ap.add_argument("--chat-ids", default="",
                    help="three token ids for the chat format: start, end, line break "
                         "(default: the reference's 151644,151645,1699)")
    ap.add_argument("--prompt-ids-file", help="a file with one request of token ids per line")
    ap.add_argument("--random-prompts", help="comma-separated lengths: one request of random ids for each")
    ap.add_argument("--random-config", help="a config.json to make random weights for")
    ap.add_argument("--write-model", help="with --random-config: the model folder to write")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--wait-for-tokens", action="store_true",
                    help="read every step's tokens before the next step is queued (by default the "
                         "next step is queued first and takes them on the device)")
    ap.add_argument("--stats", action="store_true",
                    help="at the end, print the engine's counters and where the host's time went "
                         "(LLMEngine.stats(), with the GPU time of the last step) as JSON on standard error")
    args = ap.parse_args(argv)

    if args.random_config:
        if not args.write_model:
            ap.error("--random-config needs --write-model DIR")
        from .weights.random_init import write_model_folder
        with open(args.random_config, "r", encoding="utf-8") as fh:
            config = json.load(fh)
        folder = write_model_folder(args.write_model, config, args.seed)
        print(f"wrote {folder}")
        if not args.model:
            return 0
    if not args.model:
        ap.error("--model is required")

    from .config.engine_config import EngineConfig
    from .engine.llm_engine import LLMEngine
    from .sampling.sampler import SamplingParams

    engine = LLMEngine.from_folder(args.model, EngineConfig(
        dtype=args.dtype, block_size=args.block_size, max_blocks=args.max_blocks,
        max_tokens_per_step=args.max_tokens_per_step, max_seqs=args.max_seqs, device=args.device,
        memory_fraction=args.mem_fraction, run_ahead=not args.wait_for_tokens, time_steps=args.stats))

    def report() -> None:
        if args.stats:
            print(json.dumps(engine.stats()), file=sys.stderr, flush=True)

    print(f"model ready: {len(engine.model.layers)} layers, {engine.runner.cache.num_blocks} pages "
          f"of {args.block_size} tokens", file=sys.stderr, flush=True)

    def params(i: int) -> SamplingParams:
        return SamplingParams(max_new_tokens=args.max_new_tokens, temperature=args.temperature,
                              seed=args.seed + i, ignore_eos=args.ignore_eos)

    tokenizer = None
    if args.prompt or args.text:
        from .text.vocab_tokenizer import ChatFormat, find_vocab
        tokenizer = find_vocab(args.model)
        if tokenizer is None:
            ap.error(f"--prompt and --text need a vocab.json in {args.model}")
        chat = None
        if not args.no_chat_format:
            marks = _ids(args.chat_ids)
            if len(marks) not in (0, 3):
                ap.error("--chat-ids takes three ids: start, end, line break")
            chat = ChatFormat(*marks)

    def from_text(text: str) -> List[int]:
        return chat.prompt(tokenizer, text) if chat else tokenizer.encode(text)

    prompts = [_ids(p) for p in args.prompt_ids]
    as_text = [False] * len(prompts) + [True] * len(args.prompt)
    prompts += [from_text(p) for p in args.prompt]
    if args.prompt_ids_file:
        with open(args.prompt_ids_file, "r", encoding="utf-8") as fh:
            prompts += [_ids(line) for line in fh if line.strip()]
    if args.random_prompts:
        import random
        rng = random.Random(args.seed)
        prompts += [[rng.randrange(engine.model.vocab_size) for _ in range(n)]
                    for n in _ids(args.random_prompts)]
    if prompts:
        as_text += [False] * (len(prompts) - len(as_text))
        outputs = engine.generate(prompts, [params(i) for i in range(len(prompts))])
        for out, text in zip(outputs, as_text):
            print(tokenizer.decode(out) if text else " ".join(str(t) for t in out), flush=True)
        report()
        return 0

    # interactive: a request per line, generated ids streamed as they come
    count = 0
    for line in sys.stdin:
        line = line.strip()
        if line == "exit":
            break
        if not line:
            continue
        try:
            if args.text:
                stream = tokenizer.stream()
                engine.generate([from_text(line)], [params(count)],
                                on_token=lambda _id, tok, done: print(
                                    stream.feed(tok, done), end="\n" if done else "", flush=True))
                count += 1
                continue
            prompt = _ids(line)
            engine.generate([prompt], [params(count)],
                            on_token=lambda _id, tok, done: print(tok, end="\n" if done else " ", flush=True))
        except ValueError as exc:
            print(f"error: {exc}", file=sys.stderr, flush=True)
        count += 1
    report()
    return 0


if __name__ == "__main__":
    sys.exit(main())
