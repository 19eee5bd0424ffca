"""A stand-in for the GPU model in CPU tests of the scheduler and engine loop.

It keeps what a real cache keeps, in the same places: every token written to a page slot is stored
there (with its position), and logits are computed by reading the history back through the block
table and running the plain implementation on it.  A page that is lost, shared wrongly or used again
too early therefore changes the logits, exactly as it would on the GPU.
"""
from __future__ import annotations

import numpy as np

from sprout_lm_amd.cache import CacheManager, PagedKVSpec
from tests.plain import qwen2_plain as P
from tests.test_plain import _tiny


class FakeRunner:
    device = "cpu"

    def __init__(self, block_size, num_blocks, max_sequences, prefix_caching=True, eos=(), layers=1):
        self.cfg, self.weights = _tiny(seed=9)
        self.vocab_size, self.max_positions = self.cfg["vocab_size"], 64
        self.stop_token_ids = tuple(eos)
        self.cache = CacheManager([PagedKVSpec(1, 8)] * layers, block_size, num_blocks, max_sequences, prefix_caching)
        self.slots = {}          # (page, offset) -> (token, position)
        self.steps = []          # tokens per step
        self.fed = 0             # tokens that went from one step to the next without the host seeing them
        self._memo = {}

    def logits_of(self, history) -> np.ndarray:
        key = tuple(history)
        if key not in self._memo:
            self._memo[key] = P.forward_logits(self.weights, self.cfg, list(history))[-1]
        return self._memo[key]

    def step(self, entries):
        bs = self.cache.block_size
        rows = []
        self.steps.append(sum(len(e.tokens) for e in entries))
        for e in entries:
            blocks = e.seq.blocks[0]
            for i, token in enumerate(e.tokens):
                pos = e.seq.length + i
                self.slots[(blocks[pos // bs], pos % bs)] = (token, pos)
            for w in e.want:
                history = []
                for pos in range(e.seq.length + w + 1):
                    token, stored_pos = self.slots[(blocks[pos // bs], pos % bs)]
                    assert stored_pos == pos, "a page holds another position's data"
                    history.append(token)
                rows.append(self.logits_of(history))
        for e in entries:
            self.cache.commit(e.seq, e.seq.length + len(e.tokens))
        return np.stack(rows) if rows else np.zeros((0, self.vocab_size), np.float32)

    # ---- the runner's own sampling entry points (greedy), as the engine uses them without a sampler
    def step_and_sample(self, entries, params, counters):
        return [int(np.argmax(row)) for row in self.step(entries)]

    def launch_decode(self, entries, params, counters, feed=None):
        """A step of single tokens that is "launched": computed at once here, read back by finish_decode.
        A token the host does not know yet (None) is taken from the earlier step's result, as the device does."""
        if any(len(e.tokens) != 1 or len(e.want) != 1 for e in entries):
            return None
        for i, e in enumerate(entries):
            if e.tokens[0] is None:
                assert feed is not None and feed[1][i] >= 0, "an unknown token needs a source"
                e.tokens[0] = feed[0].tokens[feed[1][i]]
                self.fed += 1
        return _Launched(self.step_and_sample(entries, params, counters))

    def finish_decode(self, launched):
        return list(launched.tokens)

    def greedy(self, prompt, steps):
        out = []
        for _ in range(steps):
            out.append(int(np.argmax(self.logits_of(list(prompt) + out))))
        return out


class _Launched:
    def __init__(self, tokens):
        self.tokens = tokens


class ArgmaxSampler:
    """First maximum wins (reference: src/runner.ts:38-42)."""

    def sample(self, logits, params, counters):
        return [int(np.argmax(row)) for row in logits]
