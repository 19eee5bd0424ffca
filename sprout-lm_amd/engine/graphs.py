"""Steps as HIP graphs.

A step in which every request brings exactly one token launches a long chain of small kernels; the
host cannot issue them as fast as the GPU runs them.  Such steps are recorded once per batch shape
into a HIP graph (through torch's capture of the current stream, which our kernels launch on) and
replayed with new values in the same device buffers.  Sampling is part of the graph, so one
descriptor upload, one graph launch and one small download make a step.

Shapes are bucketed: the number of sequences to a power of two (missing ones are filled with
one-token dummies that write no cache), the block-table width and the key splits of attention to a
power-of-two context.  Nothing in a graph depends on the values of a step.

Steps that bring portions of prompts are recorded as well once their shape comes a second time (the same
numbers of tokens and of wanted places request by request, the longest context in the same bucket): a long
prompt fed in equal portions, or a batch that decodes beside such a portion, repeats its shape step after step,
and at small model sizes the host needs as long to issue such a step's two hundred launches as the GPU to run
them.  These graphs hold no padding and no sampling; their descriptors come from the same builder as an eager
step's (`batch.step_arrays`).
"""
from __future__ import annotations

import gc
import itertools
import weakref

import numpy as np
import torch

from .. import ops
from .batch import (STEP_ARRAY_NAMES, CacheSlotView, KeptWorkspace, OwnedNames, StepContext, StepLayout, Workspace,
                    context_from, extra_step_arrays, step_arrays)


def _bucket(n: int, floor: int = 1) -> int:
    return max(floor, 1 << max(0, (n - 1)).bit_length())


class _DecodeGraph:
    """Static buffers and the recorded graph of one (sequences, context) bucket."""

    def __init__(self, runner, n_seqs: int, ctx_bucket: int):
        # the runner owns the graphs; a strong reference back would make a cycle that only the garbage
        # collector frees, at a moment of its own choosing (see _record)
        self.runner = runner if isinstance(runner, weakref.ProxyTypes) else weakref.proxy(runner)
        self.S = n_seqs
        cache = runner.cache
        self.max_blocks = [-(-ctx_bucket // g.page_tokens) for g in cache.groups]   # a table row's width, per group
        self.ctx_bucket = ctx_bucket
        S, G = n_seqs, len(cache.groups)
        # layout of the int32 staging buffer: the arrays of every step (one token a sequence: S entries each), those
        # that parts have registered, and what sampling and token feeding need
        self.extras = extra_step_arrays()
        names = list(STEP_ARRAY_NAMES) + ["x:" + name for name in self.extras] + ["counter", "temperature", "feed_source"]
        self.offsets, total = {}, 0
        for name in names:
            self.offsets[name] = (total, S)
            total += (S + 3) // 4 * 4
        self.offsets["seed"] = (total, 2 * S)
        total += (2 * S + 3) // 4 * 4
        for g in range(G):
            self.offsets[f"slots{g}"] = (total, S)
            total += (S + 3) // 4 * 4
            self.offsets[f"tables{g}"] = (total, S * self.max_blocks[g])
            total += (S * self.max_blocks[g] + 3) // 4 * 4
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=runner.device)
        view = lambda name: self.dev[self.offsets[name][0]:self.offsets[name][0] + self.offsets[name][1]]
        self.h = {name: self.host_np[o:o + n] for name, (o, n) in self.offsets.items()}
        # constant parts
        arange = np.arange(S, dtype=np.int32)
        for name in ("q_start", "logit_rows", "seq_of_token"):
            self.h[name][:] = arange
        self.h["q_len"][:] = 1
        self.h["feed_source"][:] = -1

        # buffers of its own: a graph holds their addresses, so they must never be reallocated
        ctx = StepContext(Workspace(runner.device), runner.dtype, runner.attention_kind)
        ctx.token_ids, ctx.positions, ctx.q_start = view("token_ids"), view("positions"), view("q_start")
        ctx.q_len, ctx.ctx_len, ctx.logit_rows = view("q_len"), view("ctx_len"), view("logit_rows")
        ctx.state_slots, ctx.seq_of_token = view("state_slots"), view("seq_of_token")
        ctx.extra = {name: view("x:" + name) for name in self.extras}
        empty = (self.dev[:0].view(0, 2), 0)
        every = torch.from_numpy(np.stack([arange, np.zeros_like(arange)], axis=1)).to(runner.device)
        lists = {f"tiles_multi_{t}": empty for t in ops.kernels.TILE_SIZES}
        lists.update({f"tiles_all_{t}": (every, S) for t in ops.kernels.TILE_SIZES})
        lists["decode_seqs"] = (None, S)        # every sequence brings one token, in order: no list needed
        ctx.attention = ops.AttentionBatch(ctx.q_start, ctx.q_len, ctx.ctx_len, S, lists, ctx_bucket, ctx_bucket)
        ctx.group_tables = [view(f"tables{g}").view(S, self.max_blocks[g]) for g in range(G)]
        ctx.group_slots = [view(f"slots{g}") for g in range(G)]
        ctx.n_tokens = ctx.n_seqs = ctx.n_logits = S
        ctx.max_q_len = 1
        self.ctx = ctx
        self.temperature = view("temperature").view(torch.float32)
        self.seed = view("seed").view(torch.int64)
        self.counter = view("counter")
        self.feed_source = view("feed_source")
        self.copied = None         # event: the staging buffer of the last launch has reached the device
        self.sampled = torch.zeros(S, dtype=torch.int32, device=runner.device)
        self.sample_ws = torch.empty(max(1, ops.sample_workspace_floats(S, runner.vocab_size)), dtype=torch.float32,
                                     device=runner.device)
        self.graph = None
        self.logits = None
        self._filled = -1          # number of real sequences at the last fill
        self._rows = [None] * S    # per row: which sequence and how many pages its table row holds

    def fill(self, entries, params, counters, sources=None) -> None:
        """Write this step's values into the pinned staging buffer.

        Block-table rows are rewritten only when a row's sequence or its table has changed since the last
        step (a steady decode batch gains a page every `block_size` steps; a windowed group also gives pages
        back, which the cache manager counts in the table's version).
        `sources[i] >= 0`: entry i's token is row sources[i] of an earlier step's sampled tokens, which
        the host does not know yet (its `tokens[0]` is None)."""
        cache, h, n, S = self.runner.cache, self.h, len(entries), self.S
        if self.copied is not None:
            self.copied.synchronize()      # the last launch's upload may still be reading the staging buffer
        lengths = np.fromiter((e.seq.length for e in entries), dtype=np.int32, count=n)
        h["token_ids"][:n] = [e.tokens[0] or 0 for e in entries]
        h["feed_source"][:n] = -1 if sources is None else sources
        h["positions"][:n] = lengths
        h["ctx_len"][:n] = lengths + 1
        h["state_slots"][:n] = [e.seq.state_slot for e in entries]
        h["counter"][:n] = counters
        h["temperature"].view(np.float32)[:n] = [p.temperature for p in params]
        h["seed"].view(np.int64)[:n] = [p.seed for p in params]
        if self.extras:
            first = np.arange(n, dtype=np.int32)
            layout = StepLayout(entries, lengths, np.ones(n, dtype=np.int32), first, h["state_slots"][:n], first,
                                lengths, h["token_ids"][:n])
            for name, (_, build, pad) in self.extras.items():
                h["x:" + name][:n] = np.asarray(build(layout), dtype=np.int32).reshape(-1)
                h["x:" + name][n:] = pad
        if n != self._filled:
            for name in ("token_ids", "positions", "temperature"):
                h[name][n:] = 0
            h["state_slots"][n:] = cache.spare_state_slot     # dummy rows keep their state where no request lives
            h["feed_source"][n:] = -1
            h["ctx_len"][n:] = 1
            self._rows = [None] * S
        for g in range(len(cache.groups)):
            bs, width = cache.groups[g].page_tokens, self.max_blocks[g]
            last_block = lengths // bs
            tables = h[f"tables{g}"].reshape(S, width)
            slots = h[f"slots{g}"]
            if n != self._filled:
                slots[n:] = -1
                tables[n:] = 0
            pages = np.empty(n, dtype=np.int32)
            for i, e in enumerate(entries):
                blocks = e.seq.blocks[g]
                key = (e.seq.uid, g, e.seq.table_versions[g])
                if self._rows[i] is None or self._rows[i].get(g) != key:
                    nb = min(len(blocks), width)
                    tables[i, :nb] = blocks[:nb]
                    tables[i, nb:] = -1
                    if self._rows[i] is None:
                        self._rows[i] = {}
                    self._rows[i][g] = key
                pages[i] = blocks[last_block[i]]
            slots[:n] = pages * bs + lengths % bs
        self._filled = n

    def launch(self, previous=None) -> None:
        """Upload the staging buffer and run the step; `previous`: the device tensor of sampled tokens that
        `feed_source` indexes."""
        self.dev.copy_(self.host, non_blocking=True)
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()
        if previous is not None:
            ops.feed_tokens(self.ctx.token_ids, previous, self.feed_source, self.runner.vocab_size)
        if self.graph is None:
            self._record()
        else:
            self.graph.replay()

    def _body(self):
        # What a part computes once per step for all layers (the rotation table) belongs to one step: the
        # context of a graph outlives its steps, so the table is forgotten here and its kernel is recorded
        # with the rest.  (Kept, the eager run before the capture would leave a table that the capture then
        # finds: the graph would hold no kernel for it and rotate every later step by the first step's angles.)
        self.ctx.shared.clear()
        self.logits = self.runner.forward(self.ctx)
        ops.sample(self.logits, self.sampled, self.sample_ws, self.temperature, self.seed, self.counter)

    def _record(self) -> None:
        _record(self)     # its eager run already produced this step's results


class _PortionGraph:
    """Static buffers and the recorded graph of one step shape with portions of prompts in it."""

    _uids = itertools.count(1)

    def __init__(self, runner, first, ctx_bucket: int, workspace):
        self.uid = next(self._uids)          # names this graph to the shared workspace
        self.runner = runner if isinstance(runner, weakref.ProxyTypes) else weakref.proxy(runner)
        cache = runner.cache
        self.last_used = 0
        self.table_tokens = ctx_bucket      # a block-table row holds the pages of this many tokens
        self.sizes = [a.size for a in first.arrays]
        self.offsets, total = [], 0
        for n in self.sizes:
            self.offsets.append(total)
            total += (n + 3) // 4 * 4          # every array 16-byte aligned
        self.host = torch.zeros(max(total, 4), dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(max(total, 4), dtype=torch.int32, device=runner.device)
        views = [self.dev[o:o + n].view(a.shape) for o, n, a in zip(self.offsets, self.sizes, first.arrays)]
        # Descriptors of its own; the scratch tensors are shared with the other recorded steps of this kind (they
        # run one after the other on one stream, and `workspace` never frees or moves a tensor).  The longest
        # context is known to the kernels as its bucket only (how a long walk is shared out follows it), and the
        # step has no values on the host.
        # The logits are what the caller gets: they live in a tensor of this graph's own.
        self.shared_workspace = workspace
        self.ctx = context_from(first, views, len(cache.groups), OwnedNames(workspace, ("logits",), runner.device),
                                runner.dtype, runner.attention_kind, max_decode_ctx=ctx_bucket, max_ctx=ctx_bucket)
        self.ctx.host = {}
        self.copied = None
        self.graph = None
        self.logits = None

    def fill(self, step) -> None:
        if [a.size for a in step.arrays] != self.sizes:
            raise RuntimeError("A recorded step was given arrays of another shape than it was recorded with.")
        if self.copied is not None:
            self.copied.synchronize()      # the last launch's upload may still be reading the staging buffer
        for a, o, n in zip(step.arrays, self.offsets, self.sizes):
            self.host_np[o:o + n] = a.reshape(-1)

    def launch(self) -> None:
        self.dev.copy_(self.host, non_blocking=True)
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()
        if self.graph is None:
            _record(self)
        else:
            self.graph.replay()

    def _body(self):
        self.ctx.shared.clear()            # see _DecodeGraph._body
        self.shared_workspace.owner = self.uid
        self.logits = self.runner.forward(self.ctx)


def _record(state) -> None:
    """Run `state._body` once eagerly (every workspace buffer then exists, and this step's results are there),
    then record it.

    No garbage collection while the stream is capturing: a dead cycle that holds GPU objects (an older engine's
    graphs, events, pinned buffers) would be destroyed in the middle of the capture, and what their destructors
    call is not allowed then (the process aborts).  Collect first, then hold it off."""
    state._body()
    torch.cuda.current_stream().synchronize()
    state.ctx.workspace.frozen = True
    graph = torch.cuda.CUDAGraph()
    gc.collect()
    collecting = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            state._body()
    finally:
        if collecting:
            gc.enable()
        state.ctx.workspace.frozen = False
    state.graph = graph


class DecodeGraphs:
    def __init__(self, runner, max_graphs: int = 32):
        self.runner = weakref.proxy(runner)
        self.graphs: dict[tuple, _DecodeGraph] = {}      # (sequences, context bucket) -> recorded decode step
        self.max_graphs = max_graphs
        self.replays = 0
        # steps with portions of prompts: (tokens and wanted places request by request, context bucket) -> graph
        self.portion_graphs: dict[tuple, _PortionGraph] = {}
        self.max_portion_graphs = max(4, max_graphs // 2)
        self.keep_recent = 64          # a graph used within this many such steps is not given up for a new shape
        self.portion_replays = 0
        self.portion_steps = 0
        self._sightings: dict[tuple, int] = {}
        self._portion_workspace = None

    def _context_bucket(self, longest: int) -> int:
        return min(_bucket(longest, 256), -(-self.runner.max_positions // 256) * 256)

    def _make_room(self) -> None:
        if len(self.graphs) >= self.max_graphs:
            # the least recently used graph goes; a step launched ahead may still be running from it
            torch.cuda.current_stream().synchronize()
            self.graphs.pop(next(iter(self.graphs)))

    def portion_step(self, entries, record_at: int = 2):
        """Run a step that is not one token a request from a recorded graph, if its shape has been seen
        `record_at` times (the step that reaches the count is the one recorded).  Returns the float32 logits
        at the wanted places (the graph's own tensor: valid until the same shape runs again), or None if the step
        is not taken this way: then nothing was launched.  The sequences' lengths are advanced."""
        runner = self.runner
        if not runner.parts.graph_safe_portions or not entries:
            return None
        bucket = self._context_bucket(max(e.seq.length + len(e.tokens) for e in entries))
        key = (tuple((len(e.tokens), len(e.want)) for e in entries), bucket)
        self.portion_steps += 1
        state = self.portion_graphs.pop(key, None)
        if state is None:
            seen = self._sightings.get(key, 0) + 1
            if len(self._sightings) > 4096:
                self._sightings.clear()
            self._sightings[key] = seen
            if seen < record_at:
                return None
            if len(self.portion_graphs) >= self.max_portion_graphs:
                # Recording costs as much as dozens of steps: the least recently used graph makes room only if it
                # has not run for a while.  (Shapes that take turns faster than that run eagerly.)
                oldest = next(iter(self.portion_graphs))
                if self.portion_steps - self.portion_graphs[oldest].last_used < self.keep_recent:
                    return None
                torch.cuda.current_stream().synchronize()
                self._portion_workspace.release(self.portion_graphs.pop(oldest).uid)
        step = step_arrays(entries, runner.cache, table_tokens=bucket)
        if state is None:
            if self._portion_workspace is None:
                self._portion_workspace = KeptWorkspace(runner.device)
            state = _PortionGraph(runner, step, bucket, self._portion_workspace)
        self.portion_graphs[key] = state
        state.last_used = self.portion_steps
        state.fill(step)
        state.launch()
        self.portion_replays += 1
        for e in entries:
            runner.cache.commit(e.seq, e.seq.length + len(e.tokens))
        return state.logits

    def usable(self, entries) -> bool:
        runner = self.runner
        # the parts decide: a model whose parts all launch a one-token step from device-resident values alone
        # replays, whatever its cache groups are (pages of a window, state of fixed size)
        return (runner.parts.graph_safe and len(entries) > 0
                and all(len(e.tokens) == 1 and len(e.want) == 1 for e in entries))

    def launch(self, entries, params, counters, feed=None) -> "PendingDecode":
        """Start one decode step of `entries` with sampling and return without waiting for it.

        `feed`: (an earlier, possibly unfinished PendingDecode, for every entry the row of its token among
        that step's entries or -1).  Entries with a row >= 0 carry `tokens == [None]`: the token goes from
        step to step on the device.  The sequences' lengths are advanced before the call returns.
        """
        runner = self.runner
        n = len(entries)
        S = _bucket(n)
        longest = max(e.seq.length for e in entries) + 1
        ctx_bucket = self._context_bucket(longest)
        key = (S, ctx_bucket)
        state = self.graphs.pop(key, None)
        if state is None:
            self._make_room()
            state = _DecodeGraph(runner, S, ctx_bucket)
        self.graphs[key] = state          # most recently used last
        previous, sources = (None, None) if feed is None else (feed[0].sampled, feed[1])
        state.fill(entries, params, counters, sources)
        state.launch(previous)
        self.replays += 1
        pending = PendingDecode(state.sampled, n, self._host_tokens(S), state.logits)
        for e in entries:
            runner.cache.commit(e.seq, e.seq.length + 1)
        return pending

    def run(self, entries, params, counters) -> list[int]:
        """One decode step of `entries` with sampling; returns the sampled token ids."""
        return self.launch(entries, params, counters).result()

    def _host_tokens(self, n: int) -> torch.Tensor:
        """A pinned buffer for a step's sampled tokens; a few are kept and handed out in turn (a step's
        buffer is read before the step after next is launched)."""
        if not hasattr(self, "_pinned") or self._pinned[0].numel() < n:
            self._pinned = [torch.zeros(max(n, 64), dtype=torch.int32, pin_memory=True) for _ in range(4)]
            self._turn = 0
        self._turn = (self._turn + 1) % len(self._pinned)
        return self._pinned[self._turn]


class PendingDecode:
    """A launched decode step: the sampled tokens are on their way to the host."""

    def __init__(self, sampled: torch.Tensor, n: int, host: torch.Tensor, logits: torch.Tensor | None = None):
        self.sampled, self.n = sampled, n       # the step's device buffer: valid until the same graph runs again
        self.logits = logits                    # float32 [rows of the graph, vocab], likewise; rows 0 .. n - 1 count
        self._host = host
        host[:n].copy_(sampled[:n], non_blocking=True)
        self._done = torch.cuda.Event()
        self._done.record()

    def result(self) -> list[int]:
        self._done.synchronize()
        return self._host[:self.n].tolist()
