"""The model on the device and its one step function."""
from __future__ import annotations

import json
import os

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.spec import PagedKVSpec
from ..config.base import token_id_list
from .. import ops
from ..models.plan import ModelPlan
from ..registry import build_model_plan, load_config
from ..weights.loader import load_named_tensors
from ..weights.random_init import random_tensors
from .batch import CacheSlotView, DescriptorStager, StepEntry, Workspace, build_context
from .memory import MemoryBudget, check_budget, free_device_bytes, weight_bytes

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Unsupported dtype {name}; the engine computes in bfloat16 or float32.")
        return name
    try:
        return DTYPES[name]
    except KeyError:
        raise ValueError(f"Unknown dtype {name!r}; choose bfloat16 or float32.") from None


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("No GPU is visible: the engine runs its HIP kernels on an AMD GPU and has no CPU path.")
    return torch.device("cuda", torch.cuda.current_device())


class ModelRunner:
    """Weights, cache pools and workspace of one model, and `step`.

    `step` runs exactly the tokens it is given, as one batch, reading earlier tokens from the
    cache, and returns float32 logits at the wanted places.
    """

    def __init__(self, plan: ModelPlan, tensors: dict, dtype: torch.dtype, device, block_size: int, num_blocks: int,
                 max_sequences: int, prefix_caching: bool = False, stop_token_ids=None, use_graphs: bool = True,
                 budget: MemoryBudget | None = None, parts=None):
        """`tensors`: the plan's tensors on the device, by checkpoint name (the dict is emptied as parts take
        them); None: `parts` hold their tensors already (`with_pool_of_its_own`).  The cache pools are counted
        against the free device memory before they are allocated."""
        self.plan, self.dtype, self.device = plan, dtype, device
        self.parts = parts if parts is not None else plan.instantiate()
        self.budget = budget or MemoryBudget()
        # whether pages of a common prefix may be shared is the architecture's word (the plan), then the caller's
        self.cache = CacheManager(self.parts.cache_slot_specs, block_size, num_blocks, max_sequences,
                                  prefix_caching and self.parts.prefix_sharing)
        if torch.device(device).type == "cuda":
            check_budget(0, self.cache.storage_bytes(dtype.itemsize), free_device_bytes(device), self.budget,
                         "cache pools (the weights are resident already)")
        if tensors is not None:
            self.parts.bind(tensors, device, dtype)
        self.cache.attach_storage(dtype, device)
        self.workspace = Workspace(device)
        self.stager = DescriptorStager(device)
        self.stop_token_ids = tuple(stop_token_ids if stop_token_ids is not None else plan.eos_token_ids)
        self.attention_kind = 1 if dtype == torch.float32 else 0
        self.vocab_size, self.hidden_size, self.max_positions = plan.vocab_size, plan.hidden_size, plan.max_positions
        self.use_graphs = use_graphs
        self.record_portions = True      # steps with portions of prompts are recorded too, once their shape recurs
        self.load_notes: list[str] = []    # what the loader saw and left alone (tensors nobody asked for)
        self._graphs = None
        self._sampler = None

    # ------------------------------------------------------------------ construction
    @staticmethod
    def preflight(parts, dtype: torch.dtype, device, block_size: int, num_blocks: int, max_sequences: int,
                  budget: MemoryBudget, stored: dict | None = None) -> tuple[int, int]:
        """Count the weights and the cache pools of a model that is not loaded yet against the device's free
        memory; raises MemoryBudgetError if they do not fit.  Returns (weight bytes, pool bytes)."""
        weights = weight_bytes(parts.expected_tensors(), dtype, stored)
        pools = CacheManager.pool_bytes(parts.cache_slot_specs, block_size, num_blocks, max_sequences, dtype.itemsize)
        check_budget(weights, pools, free_device_bytes(device), budget)
        return weights, pools

    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", strict_tensors: bool = False, weight_limit_mib: int = 0,
                    reserve_mib: int | None = None, **cache_options) -> "ModelRunner":
        """`strict_tensors`: tensors in the checkpoint that the model does not ask for are an error (by
        default they are left unread, as the reference leaves them: src/safetensors.ts:70-83)."""
        device = require_gpu()
        dtype = parse_dtype(dtype)
        config = load_config(folder)
        plan = build_model_plan(config)
        parts = plan.instantiate()
        budget = MemoryBudget(weight_limit_mib, MemoryBudget().reserve_mib if reserve_mib is None else reserve_mib)
        sizes = {k: cache_options[k] for k in ("block_size", "num_blocks", "max_sequences")}
        notes: list[str] = []
        tensors = load_named_tensors(
            folder, parts.expected_tensors(), set(plan.ignorable_tensors), dtype, device, strict=strict_tensors,
            notes=notes, before_read=lambda stored: cls.preflight(parts, dtype, device, budget=budget, stored=stored, **sizes))
        runner = cls(plan, tensors, dtype, device, stop_token_ids=stop_ids_of_folder(folder, plan), budget=budget,
                     parts=parts, **cache_options)
        runner.load_notes = notes
        return runner

    @classmethod
    def from_config(cls, config, seed: int, dtype="bfloat16", weight_limit_mib: int = 0, reserve_mib: int | None = None,
                    **cache_options) -> "ModelRunner":
        """Random weights drawn on the device (for benchmarks; a model folder is not written)."""
        device = require_gpu()
        dtype = parse_dtype(dtype)
        plan = build_model_plan(config)
        parts = plan.instantiate()
        budget = MemoryBudget(weight_limit_mib, MemoryBudget().reserve_mib if reserve_mib is None else reserve_mib)
        cls.preflight(parts, dtype, device, budget=budget,
                      **{k: cache_options[k] for k in ("block_size", "num_blocks", "max_sequences")})
        tensors = random_tensors(parts.expected_tensors(), seed, dtype=dtype, device=device)
        return cls(plan, tensors, dtype, device, budget=budget, parts=parts, **cache_options)

    def with_pool_of_its_own(self, block_size: int, num_blocks: int, max_sequences: int, prefix_caching: bool = False,
                             use_graphs: bool = True) -> "ModelRunner":
        """A second runner over the same weights with a cache pool, workspace and recorded graphs of its own (a
        small pool beside a large one, say).  The two must not step at the same time: the parts are shared."""
        other = ModelRunner(self.plan, None, self.dtype, self.device, block_size, num_blocks, max_sequences,
                            prefix_caching, self.stop_token_ids, use_graphs, self.budget, parts=self.parts)
        other.load_notes = list(self.load_notes)
        return other

    # ------------------------------------------------------------------ the step
    def _slot_views(self, ctx, call_index: int) -> dict:
        """What the parts of one call of the run order get for their caches: part name -> view, or -> a dict of
        views where the part asked for several things by name."""
        views: dict = {}
        for key, (slot, writes) in self.parts.call_slots[call_index].items():
            kind, g, index = self.cache.slot_location[slot]
            if kind == "paged":
                group = self.cache.groups[g]
                view = CacheSlotView(writes, k=group.k[index], v=group.v[index], block_tables=ctx.group_tables[g],
                                     slot_mapping=ctx.group_slots[g], page_size=group.page_tokens)
            else:
                view = CacheSlotView(writes, state=self.cache.state_groups[g].data[index])
            name, _, sub = key.partition(".")
            if sub:
                views.setdefault(name, {})[sub] = view
            else:
                views[name] = view
        return views

    def validate(self, entries: list[StepEntry]) -> None:
        seen = set()
        for e in entries:
            if id(e.seq) in seen:
                raise ValueError("A request appears twice in one step.")
            seen.add(id(e.seq))
            if e.seq.released:
                raise ValueError("A request's cache was released before the step.")
            n = len(e.tokens)
            if n == 0:
                raise ValueError("A step entry brings no tokens.")
            if n > 32:     # a long portion: checked as one array (a list that is not all integers has another kind)
                ids = np.asarray(e.tokens)
                bad = ids.dtype.kind not in "iu" or ids.ndim != 1 or int(ids.min()) < 0 or int(ids.max()) >= self.vocab_size
            else:
                bad = any(not isinstance(t, int) or isinstance(t, bool) or t < 0 or t >= self.vocab_size for t in e.tokens)
            if bad:
                raise ValueError(f"Token ids must be integers in [0, {self.vocab_size}).")
            if e.seq.length + n > self.max_positions:
                raise ValueError(f"Position {e.seq.length + n - 1} is beyond the model's {self.max_positions} positions.")
            if any(not isinstance(w, int) or w < 0 or w >= n for w in e.want):
                raise ValueError("Wanted logit places must index the entry's own tokens.")
            for gi, needed in enumerate(self.cache.pages_needed(e.seq, e.seq.length + n)):
                if needed:
                    raise ValueError("Pages for the entry's tokens were not reserved before the step.")

    def validate_decode(self, entries: list[StepEntry], sources=None) -> None:
        """The checks of `validate` for a step of single tokens, in one pass.  An entry whose token is still
        on the device (`sources[i] >= 0`) brings None in its place."""
        seen = set()
        sizes, limit, vocab = [g.page_tokens for g in self.cache.groups], self.max_positions, self.vocab_size
        for i, e in enumerate(entries):
            seq, token = e.seq, e.tokens[0]
            if token is None and sources is not None and sources[i] >= 0:
                token = 0
            if id(seq) in seen:
                raise ValueError("A request appears twice in one step.")
            seen.add(id(seq))
            if seq.released:
                raise ValueError("A request's cache was released before the step.")
            if not isinstance(token, int) or token < 0 or token >= vocab:
                raise ValueError(f"Token ids must be integers in [0, {vocab}).")
            if seq.length >= limit:
                raise ValueError(f"Position {seq.length} is beyond the model's {limit} positions.")
            if e.want[0] != 0:
                raise ValueError("Wanted logit places must index the entry's own tokens.")
            for bs, blocks in zip(sizes, seq.blocks):
                if len(blocks) < seq.length // bs + 1:
                    raise ValueError("Pages for the entry's tokens were not reserved before the step.")

    def step(self, entries: list[StepEntry]) -> torch.Tensor:
        """Run one batch; returns float32 logits [number of wanted places, vocab] on the device.

        The sequences' lengths are advanced (and pages that a window has passed are given back)
        before the call returns; the kernels may still be running on the stream.
        """
        self.validate(entries)
        return self._step_checked(entries)

    def _step_checked(self, entries: list[StepEntry]) -> torch.Tensor:
        ctx = build_context(entries, self.cache, self.stager, self.workspace, self.dtype, self.attention_kind)
        logits = self.forward(ctx)
        for e in entries:
            self.cache.commit(e.seq, e.seq.length + len(e.tokens))
        return logits

    def step_and_sample(self, entries: list[StepEntry], params, counters) -> list[int]:
        """One step plus sampling at every wanted place; returns the sampled token ids on the host.

        Steps in which every request brings one token are replayed from a recorded HIP graph; so are other
        steps whose shape comes again and again (`step_recorded`).
        """
        from ..sampling.sampler import Sampler
        pending = self.launch_decode(entries, params, counters)
        if pending is not None:
            return self.finish_decode(pending)
        if self._sampler is None:
            self._sampler = Sampler(self.device, self.vocab_size)
        self.validate(entries)
        logits = self._recorded_checked(entries, 2)
        if logits is None:
            logits = self._step_checked(entries)
        return self._sampler.sample(logits, params, counters)

    def step_recorded(self, entries: list[StepEntry], record_at: int = 2):
        """`step` from a recorded graph of the step's shape, where there is one or the shape has now come
        `record_at` times; None otherwise (nothing has been run then).  The logits lie in a tensor of that graph's
        own: they stay until a step of the same shape runs again, whatever other steps run meanwhile."""
        if not self.use_graphs or not self.record_portions or not self.parts.graph_safe_portions:
            return None
        self.validate(entries)
        return self._recorded_checked(entries, record_at)

    def _recorded_checked(self, entries: list[StepEntry], record_at: int):
        if not self.use_graphs or not self.record_portions or not self.parts.graph_safe_portions:
            return None
        if self._graphs is None:
            from .graphs import DecodeGraphs
            self._graphs = DecodeGraphs(self)
        return self._graphs.portion_step(entries, record_at)

    def launch_decode(self, entries: list[StepEntry], params, counters, feed=None):
        """Start a step in which every request brings one token, without waiting for its result.

        Returns a handle for `finish_decode`, or None if the step cannot run from a recorded graph (then
        nothing has been launched).  `feed`: (handle of an earlier step, row of each entry's token among that
        step's entries or -1): tokens the host has not seen go from step to step on the device.
        """
        if not self.use_graphs:
            return None
        if self._graphs is None:
            from .graphs import DecodeGraphs
            self._graphs = DecodeGraphs(self)
        if not self._graphs.usable(entries):
            return None
        self.validate_decode(entries, None if feed is None else feed[1])
        return self._graphs.launch(entries, params, counters, feed)

    def finish_decode(self, pending) -> list[int]:
        """Wait for a launched decode step; returns its sampled token ids."""
        from ..sampling.sampler import NonFiniteLogits
        tokens = pending.result()
        if any(t < 0 or t >= self.vocab_size for t in tokens):
            raise NonFiniteLogits("Non-finite logits: the model produced NaN or infinity.")
        return tokens

    def forward(self, ctx) -> torch.Tensor:
        T, H = ctx.n_tokens, self.hidden_size
        with ops.stream_scope():       # one stream lookup for the step's launches
            residual = ctx.buffer("residual", (T, H), torch.float32)
            self.parts.embedding.forward(ctx, ctx.token_ids, residual)
            for i, call in enumerate(self.plan.schedule):
                self.parts.blocks[call.layer].forward(ctx, residual, self._slot_views(ctx, i))
            n = ctx.n_logits
            logits = ctx.buffer("logits", (n, self.vocab_size), torch.float32)
            if n:
                normed = ctx.buffer("final_normed", (n, H), self.dtype)
                self.parts.final_norm.forward(ctx, residual, normed, rows=ctx.logit_rows)
                self.parts.head.forward(ctx, normed, logits)
        return logits

    # ------------------------------------------------------------------ sizes
    def kv_bytes_per_token(self) -> int:
        size = torch.empty((), dtype=self.dtype).element_size()
        return sum(2 * s.kv_heads * s.head_dim * size for s in self.parts.cache_slot_specs if isinstance(s, PagedKVSpec))


def stop_ids_of_folder(folder: str, plan: ModelPlan) -> tuple[int, ...]:
    """generation_config.json's eos_token_id replaces the configuration's (reference: src/qwen.ts:124-128)."""
    path = os.path.join(folder, "generation_config.json")
    if os.path.exists(path):
        with open(path) as f:
            generation = json.load(f)
        if isinstance(generation, dict) and generation.get("eos_token_id") is not None:
            return token_id_list(generation["eos_token_id"], plan.vocab_size, "generation_config eos_token_id")
    return tuple(plan.eos_token_ids)
