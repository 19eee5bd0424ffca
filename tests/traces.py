"""Builders of replay traces: the same requests cut into steps in different ways.

A trace is a list of step records in the format that `bin/trace_run` reads.  `expected` pairs every
wanted logits row with (request id, position), so that any cut can be compared with the plain
implementation's whole-sequence logits.
"""
from __future__ import annotations

import numpy as np


class Trace:
    def __init__(self):
        self.steps: list[dict] = []
        self.expected: list[list[tuple[str, int]]] = []   # per step: (request, position) of each wanted row

    def add(self, entries, end=()):
        """entries: list of (request id, first position, tokens, wanted offsets)."""
        step = {"step": len(self.steps), "entries": [], "end": list(end)}
        rows = []
        for rid, first, tokens, want in entries:
            step["entries"].append({"id": rid, "tokens": [int(t) for t in tokens], "want": [int(w) for w in want]})
            rows += [(rid, first + w) for w in want]
        self.steps.append(step)
        self.expected.append(rows)


def whole(requests: dict[str, list[int]]) -> Trace:
    """Each request alone, its whole prompt in one step, logits everywhere."""
    t = Trace()
    for rid, tokens in requests.items():
        t.add([(rid, 0, tokens, range(len(tokens)))], end=[rid])
    return t


def tail_decoded(requests: dict[str, list[int]], tail: int = 32) -> Trace:
    """Most of a request in one step, its last `tail` tokens one by one."""
    t = Trace()
    for rid, tokens in requests.items():
        head = max(1, len(tokens) - tail)
        t.add([(rid, 0, tokens[:head], [head - 1])])
        for p in range(head, len(tokens)):
            t.add([(rid, p, tokens[p:p + 1], [0])], end=[rid] if p == len(tokens) - 1 else [])
        if head == len(tokens):
            t.add([], end=[rid])
    return t


def portions(requests: dict[str, list[int]], sizes=(16, 7, 5, 3, 2, 2, 9, 4, 2, 11)) -> Trace:
    """Each request alone in portions of changing size, down to two tokens; logits at every position."""
    t = Trace()
    for rid, tokens in requests.items():
        p, i = 0, 0
        while p < len(tokens):
            n = min(sizes[i % len(sizes)], len(tokens) - p)
            i += 1
            t.add([(rid, p, tokens[p:p + n], range(n))], end=[rid] if p + n == len(tokens) else [])
            p += n
    return t


def mixed(requests: dict[str, list[int]], seed: int, max_live: int = 4, tail: int = 12) -> Trace:
    """Up to `max_live` requests at a time: portions of some beside single decoded tokens of others.

    Every request is fed in random portions (2..13 tokens) until `tail` tokens remain, then token by
    token; now and then a request sits a step out.  New requests start as old ones end, so with a
    small pool their pages are the ones just given back.
    """
    rng = np.random.default_rng(seed)
    t = Trace()
    waiting = list(requests.items())
    live: dict[str, int] = {}      # request -> tokens fed so far
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            tokens, p = requests[rid], live[rid]
            if len(live) > 1 and rng.random() < 0.15:
                continue          # left out of this step
            left = len(tokens) - p
            n = 1 if left <= tail else int(min(rng.integers(2, 14), left - tail))
            want = [n - 1] if n > 1 and rng.random() < 0.7 else list(range(n)) if n == 1 else [0, n - 1]
            entries.append((rid, p, tokens[p:p + n], want))
            live[rid] = p + n
            if live[rid] == len(tokens):
                ended.append(rid)
                del live[rid]
        t.add(entries, end=ended)
    return t
