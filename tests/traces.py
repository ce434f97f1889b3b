"""Traces: the same requests cut into steps in different ways.  A trace is a list of steps;
a step is ``(entries, end)`` with entries ``(request, tokens, want)``.  Every function returns
(steps, expect) where ``expect[(request, position)]`` marks a position whose logits are asked
for, so that results can be compared with a whole-sequence run."""
import random


def whole(prompts):
    """Each request alone and whole, one step each; logits at every position."""
    steps = []
    for name, ids in prompts.items():
        steps.append(([(name, list(ids), list(range(len(ids))))], [name]))
    return steps


def tail_decode(prompts, tail=32):
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for name, ids in prompts.items():
        cut = max(1, len(ids) - tail)
        steps.append(([(name, list(ids[:cut]), list(range(cut)))], [name] if cut == len(ids) else []))
        for i in range(cut, len(ids)):
            steps.append(([(name, [ids[i]], [0])], [name] if i == len(ids) - 1 else []))
    return steps


def chunked(prompts, sizes=(7, 2, 16, 3, 2, 5, 11, 2, 33, 4)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for name, ids in prompts.items():
        pos, k = 0, 0
        while pos < len(ids):
            n = min(sizes[k % len(sizes)], len(ids) - pos)
            k += 1
            last = pos + n >= len(ids)
            steps.append(([(name, list(ids[pos:pos + n]), list(range(n)))], [name] if last else []))
            pos += n
    return steps


def mixed(prompts, seed=0, max_live=4, decode_tail=12):
    """Up to ``max_live`` live requests: portions of some beside single decoded tokens of
    others.  Each request is fed in random portions until ``decode_tail`` tokens are left,
    which then go one per step; requests start as others end."""
    rng = random.Random(seed)
    order = list(prompts)
    waiting = list(order)
    live = {}          # name -> position fed so far
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for name in list(live):
            ids = prompts[name]
            pos = live[name]
            if rng.random() < 0.15 and len(live) > 1:
                continue                      # left out of this step, goes on later
            left = len(ids) - pos
            if left <= decode_tail:
                n = 1
            else:
                n = min(left - decode_tail, rng.choice((2, 3, 5, 8, 13, 21, 40)))
            entries.append((name, list(ids[pos:pos + n]), list(range(n))))
            live[name] = pos + n
            if live[name] >= len(ids):
                end.append(name)
                del live[name]
        if entries:
            steps.append((entries, end))
    return steps


def max_live_tokens(steps, page=64):
    """The most tokens that live requests hold at any time, each rounded up to ``page``."""
    held, peak = {}, 0
    for entries, end in steps:
        for name, tokens, _ in entries:
            held[name] = held.get(name, 0) + len(tokens)
        peak = max(peak, sum(-(-n // page) * page for n in held.values()))
        for name in end:
            held.pop(name, None)
    return peak
