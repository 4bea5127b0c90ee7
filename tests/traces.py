"""Ways of cutting the same requests into steps.  A trace is a list of steps;
a step is ``(entries, ends)`` with entries ``(rid, start, n)``: request ``rid``
brings its tokens ``start .. start+n-1``.  Every fed token's logits are wanted."""

from __future__ import annotations

import random
from typing import Dict, List, Sequence, Tuple

Step = Tuple[List[Tuple[str, int, int]], List[str]]


def whole(lengths: Dict[str, int]) -> List[Step]:
    """Each request alone and whole."""
    return [([(rid, 0, n)], [rid]) for rid, n in lengths.items()]


def tail(lengths: Dict[str, int], n_tail: int = 32) -> List[Step]:
    """Most of it in one step, the last ``n_tail`` tokens one by one."""
    steps: List[Step] = []
    for rid, n in lengths.items():
        head = max(1, n - n_tail)
        steps.append(([(rid, 0, head)], []))
        for p in range(head, n):
            steps.append(([(rid, p, 1)], []))
        steps[-1] = (steps[-1][0], [rid])
    return steps


def chunks(lengths: Dict[str, int], sizes: Sequence[int] = (7, 2, 13, 3, 1, 29, 2, 64, 5)) -> List[Step]:
    """Portions of changing size, down to two tokens (and one)."""
    steps: List[Step] = []
    for rid, n in lengths.items():
        p, i = 0, 0
        while p < n:
            c = min(sizes[i % len(sizes)], n - p)
            steps.append(([(rid, p, c)], [rid] if p + c == n else []))
            p, i = p + c, i + 1
    return steps


def mixed(lengths: Dict[str, int], max_live: int = 4, seed: int = 0, prompt_frac: float = 0.6,
          budget: int = 48) -> List[Step]:
    """Up to ``max_live`` live requests; portions of some prompts beside single
    tokens of requests that are past their "prompt" (the first ``prompt_frac``
    of their tokens), under a token budget per step; a finished request's pages
    go to the next one waiting."""
    rng = random.Random(seed)
    waiting = list(lengths)
    live: Dict[str, int] = {}
    steps: List[Step] = []
    while waiting or live:
        while waiting and len(live) < max_live:
            live[waiting.pop(0)] = 0
        entries, ends, left = [], [], budget
        order = list(live)
        rng.shuffle(order)
        for rid in order:
            n, p = lengths[rid], live[rid]
            n_prompt = max(1, int(n * prompt_frac))
            if p >= n_prompt:
                c = 1
            else:
                c = min(n_prompt - p, rng.choice([2, 3, 5, 8, 17, 32]))
            if rng.random() < 0.15 and len(order) > 1:
                continue  # a request may be left out of a step and go on later
            if c > left:
                if left < 2:
                    continue
                c = left if p < n_prompt else 1
            entries.append((rid, p, c))
            left -= c
            live[rid] = p + c
            if p + c == n:
                ends.append(rid)
        for rid in ends:
            del live[rid]
        if entries:
            steps.append((entries, ends))
    return steps


def max_live_tokens(trace: List[Step], round_to: int = 64) -> int:
    """Most tokens live requests hold at any time, each rounded up."""
    held: Dict[str, int] = {}
    worst = 0
    for entries, ends in trace:
        for rid, start, n in entries:
            held[rid] = start + n
        worst = max(worst, sum(-(-v // round_to) * round_to for v in held.values()))
        for rid in ends:
            held.pop(rid, None)
    return worst


def many_decoding_together(prompt_lens: Dict[str, int], n_decode: int, seed: int = 0, budget: int = 96,
                           max_per_step: int = 6) -> List[Step]:
    """All requests become live, their prompts fed in portions of changing size (a few requests a
    step, under a token budget); then every request decodes, all of them in every step, for
    ``n_decode`` steps, and all end together."""
    rng = random.Random(seed)
    fed = {rid: 0 for rid in prompt_lens}
    steps: List[Step] = []
    while any(fed[r] < n for r, n in prompt_lens.items()):
        entries, left = [], budget
        todo = [r for r, n in prompt_lens.items() if fed[r] < n]
        rng.shuffle(todo)
        for rid in todo[:max_per_step]:
            c = min(prompt_lens[rid] - fed[rid], rng.choice([2, 3, 7, 16, 33, 64]), left)
            if c < 1:
                break
            entries.append((rid, fed[rid], c))
            fed[rid] += c
            left -= c
        steps.append((entries, []))
    for s in range(n_decode):
        steps.append(([(rid, n + s, 1) for rid, n in prompt_lens.items()],
                      list(prompt_lens) if s == n_decode - 1 else []))
    return steps
