"""The batch of one step: what parts see while they run.

A step holds, for every request in it, the next tokens of that request (a portion of its prompt or
one decoded token).  All tokens are laid out flat, request after request.  The integer arrays that
the kernels need are packed into one host buffer and copied to the device in one transfer.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from .. import ops


@dataclass
class StepEntry:
    """One request's share of a step: its cache, its next tokens, and where logits are wanted."""

    seq: object                 # cache.SequenceCache
    tokens: list
    want: list                  # indices into `tokens`


@dataclass
class CacheSlotView:
    """What a mixer gets for its cache slot in this step."""

    writes: bool
    k: torch.Tensor | None = None            # [pages, kv_heads, page_size, head_dim]
    v: torch.Tensor | None = None            # [pages, kv_heads, head_dim, page_size]
    block_tables: torch.Tensor | None = None  # int32 [sequences, max_blocks]
    slot_mapping: torch.Tensor | None = None  # int32 [tokens]: page * page_size + offset
    state: torch.Tensor | None = None         # [max_sequences, *shape] for a fixed-size state slot
    page_size: int = 0


class Workspace:
    """Named scratch tensors that live across steps and grow on demand."""

    def __init__(self, device):
        self.device = device
        self.frozen = False      # while a graph is recorded nothing may be allocated
        self._flat: dict[tuple[str, torch.dtype], torch.Tensor] = {}

    def get(self, name: str, shape, dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= s
        key = (name, dtype)
        flat = self._flat.get(key)
        if flat is None or flat.numel() < n:
            if self.frozen:
                raise RuntimeError(f"Workspace buffer {name!r} would grow while a graph is recorded.")
            flat = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._flat[key] = flat
        return flat[:n].view(shape)


class KeptWorkspace(Workspace):
    """Scratch tensors for recorded graphs that share them: a graph holds the addresses it was recorded with, so
    a tensor is never moved, and freed only when every graph that used it has been given up (`release`); a request
    that none of a name's tensors can hold gets a further one.  `owner` names the graph that is asking."""

    def __init__(self, device):
        super().__init__(device)
        self._kept: dict[tuple[str, torch.dtype], list[torch.Tensor]] = {}
        self._users: dict[int, set] = {}      # id(tensor) -> owners that were handed it
        self.owner = None

    def get(self, name: str, shape, dtype) -> torch.Tensor:
        n = 1
        for s in shape:
            n *= s
        fitting = [t for t in self._kept.get((name, dtype), ()) if t.numel() >= n]
        if fitting:
            flat = min(fitting, key=lambda t: t.numel())
        else:
            if self.frozen:
                raise RuntimeError(f"Workspace buffer {name!r} would grow while a graph is recorded.")
            flat = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._kept.setdefault((name, dtype), []).append(flat)
        self._users.setdefault(id(flat), set()).add(self.owner)
        return flat[:n].view(shape)

    def release(self, owner) -> None:
        """`owner`'s graph is gone (and the stream has been waited for): free what no other graph uses."""
        for key, kept in list(self._kept.items()):
            still = []
            for flat in kept:
                users = self._users.get(id(flat), set())
                users.discard(owner)
                if users:
                    still.append(flat)
                else:
                    self._users.pop(id(flat), None)
            if still:
                self._kept[key] = still
            else:
                del self._kept[key]

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for kept in self._kept.values() for t in kept)


class OwnedNames:
    """A workspace that keeps the named buffers for itself and asks `shared` for every other: what a recorded step
    returns to its caller (the logits) must not be overwritten by the next recorded step of another shape."""

    def __init__(self, shared: Workspace, own: tuple, device):
        self.shared, self.own, self.private = shared, own, Workspace(device)

    @property
    def frozen(self):
        return self.shared.frozen

    @frozen.setter
    def frozen(self, value):
        self.shared.frozen = self.private.frozen = value

    def get(self, name: str, shape, dtype) -> torch.Tensor:
        return (self.private if name in self.own else self.shared).get(name, shape, dtype)


class StepContext:
    def __init__(self, workspace: Workspace, act_dtype, attention_kind: int = 0):
        self.workspace = workspace
        self.act_dtype = act_dtype
        self.attention_kind = attention_kind
        self.n_tokens = self.n_seqs = self.n_logits = 0
        self.max_q_len = 0
        self.token_ids = self.positions = self.q_start = self.q_len = self.ctx_len = None
        self.logit_rows = self.state_slots = self.seq_of_token = None
        self.attention = None   # ops.AttentionBatch of this step
        self.group_tables: list[torch.Tensor] = []
        self.group_slots: list[torch.Tensor] = []
        self.extra = {}  # arrays that parts have registered (register_step_array), by name, on the device
        self.host = {}   # the same arrays on the host (numpy), for parts that plan on the CPU
        self.shared = {}   # what a part computes once per step for all layers (key chosen by the part)

    def buffer(self, name: str, shape, dtype) -> torch.Tensor:
        return self.workspace.get(name, shape, dtype)

class DescriptorStager:
    """Pinned host buffers, used in turn, through which a step's integer arrays reach the device."""

    def __init__(self, device, depth: int = 4):
        self.device = device
        self.depth = depth
        self._host = [None] * depth
        self._dev = [None] * depth
        self._events = [None] * depth
        self._turn = 0

    def upload(self, arrays: list[np.ndarray]) -> list[torch.Tensor]:
        """Copy the int32 arrays to the device in one transfer; returns a device view per array."""
        sizes = [a.size for a in arrays]
        offsets, total = [], 0
        for n in sizes:
            offsets.append(total)
            total += (n + 3) // 4 * 4     # keep every array 16-byte aligned
        i = self._turn
        self._turn = (self._turn + 1) % self.depth
        if self._events[i] is not None:
            self._events[i].synchronize()
        if self._host[i] is None or self._host[i].numel() < total:
            cap = max(4096, 1 << (max(total, 1) - 1).bit_length())
            self._host[i] = torch.empty(cap, dtype=torch.int32, pin_memory=True)
            self._dev[i] = torch.empty(cap, dtype=torch.int32, device=self.device)
        host = self._host[i].numpy()
        for a, off, n in zip(arrays, offsets, sizes):
            host[off:off + n] = a.reshape(-1)
        self._dev[i][:total].copy_(self._host[i][:total], non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        self._events[i] = event
        return [self._dev[i][off:off + n].view(a.shape) for a, off, n in zip(arrays, offsets, sizes)]


# The integer arrays of every step, in staging order; each has one entry per token or per sequence.  The recorded
# decode steps lay their static buffers out from this list too (engine.graphs), so an array is named once.
STEP_ARRAY_NAMES = ("token_ids", "positions", "q_start", "q_len", "ctx_len", "logit_rows", "state_slots", "seq_of_token")

# Arrays that parts add to every step: name -> (per, function of a StepLayout, value of padded rows).
_EXTRA_ARRAYS: dict[str, tuple[str, object, int]] = {}


def register_step_array(name: str, per: str, build, pad: int = 0) -> None:
    """Add an int32 array to every step from now on: `build(layout)` returns one entry per token (`per` "token")
    or per sequence ("sequence") of the step described by `layout` (a StepLayout).  Parts find its device copy
    in `ctx.extra[name]`, in eager steps and recorded ones alike; rows that a recorded step adds as padding hold
    `pad`.  (In a recorded step of single tokens a token id that is still on the device reads 0 in the layout.)
    Registered once, by the module that defines the part that needs it, before the model is built."""
    if per not in ("token", "sequence"):
        raise ValueError("A step array has one entry per 'token' or per 'sequence'.")
    _EXTRA_ARRAYS[name] = (per, build, int(pad))


def unregister_step_array(name: str) -> None:
    _EXTRA_ARRAYS.pop(name, None)


def extra_step_arrays() -> dict:
    return dict(_EXTRA_ARRAYS)


@dataclass
class StepLayout:
    """A step as the builders of its arrays see it: per sequence the first position, the number of new tokens,
    the start of its tokens in the flat order and its state slot; per token its sequence, position and id."""

    entries: list
    first_pos: np.ndarray
    q_len: np.ndarray
    q_start: np.ndarray
    state_slots: np.ndarray
    seq_of_token: np.ndarray
    positions: np.ndarray
    token_ids: np.ndarray


def _extras(layout: StepLayout) -> list:
    out = []
    for name, (per, build, _) in _EXTRA_ARRAYS.items():
        array = np.ascontiguousarray(build(layout), dtype=np.int32).reshape(-1)
        want = len(layout.token_ids) if per == "token" else len(layout.q_len)
        if array.size != want:
            raise ValueError(f"Step array {name!r} has {array.size} entries for {want} {per}s.")
        out.append(("x:" + name, array))
    return out


@dataclass
class StepArrays:
    """A step's integer arrays on the host, in the order in which they are staged, and what the step's kernels
    need to know of them.  One builder serves the eager step and the recorded ones."""

    names: list            # one name per array, in staging order
    arrays: list           # numpy int32 arrays
    lists: dict            # attention work lists by name (also part of `arrays`)
    n_tokens: int
    n_seqs: int
    n_logits: int
    max_q_len: int
    max_decode_ctx: int
    max_ctx: int
    mean_walk: int
    host: dict

    def named(self, name: str):
        return self.arrays[self.names.index(name)]


def step_arrays(entries: list[StepEntry], cache, table_tokens: int | None = None) -> StepArrays:
    """Lay the entries out flat: token ids, positions, per-sequence start / length / context, the places of
    wanted logits, state slots, the arrays that parts have registered, the attention work lists, and per cache
    group the block tables (a row holds the pages of `table_tokens` tokens, by default as many as the longest
    table) and the cache slot of every token.

    Each entry's sequence must already hold pages for its new tokens (CacheManager.reserve).
    """
    q_lens = [len(e.tokens) for e in entries]
    starts = np.zeros(len(entries), dtype=np.int32)
    if entries:
        starts[1:] = np.cumsum(q_lens[:-1])
    T = int(sum(q_lens))
    first_pos = np.asarray([e.seq.length for e in entries], dtype=np.int32)
    q_len = np.asarray(q_lens, dtype=np.int32)
    ctx_len = first_pos + q_len
    token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries]) if T else np.zeros(0, np.int32)
    seq_of_token = np.repeat(np.arange(len(entries), dtype=np.int32), q_len)
    positions = (np.arange(T, dtype=np.int32) - starts[seq_of_token] + first_pos[seq_of_token]).astype(np.int32)
    rows = [starts[s] + w for s, e in enumerate(entries) for w in e.want]
    logit_rows = np.asarray(rows, dtype=np.int32)
    state_slots = np.asarray([e.seq.state_slot for e in entries], dtype=np.int32)

    core = {"token_ids": token_ids, "positions": positions, "q_start": starts, "q_len": q_len, "ctx_len": ctx_len,
            "logit_rows": logit_rows, "state_slots": state_slots, "seq_of_token": seq_of_token}
    names = list(STEP_ARRAY_NAMES)
    arrays = [core[name] for name in names]
    if _EXTRA_ARRAYS:
        for name, array in _extras(StepLayout(entries, first_pos, q_len, starts, state_slots, seq_of_token, positions,
                                              token_ids)):
            names.append(name)
            arrays.append(array)
    lists = ops.attention_lists(q_lens)
    for name in sorted(lists):
        names.append(name)
        arrays.append(lists[name])
    for gi, group in enumerate(cache.groups):
        bs = group.page_tokens
        width = -(-table_tokens // bs) if table_tokens else max(1, max((len(e.seq.blocks[gi]) for e in entries), default=1))
        tables = np.full((len(entries), width), -1, dtype=np.int32)
        slots = np.full(T, -1, dtype=np.int32)
        for s, e in enumerate(entries):
            blocks = e.seq.blocks[gi][:width]
            tables[s, :len(blocks)] = blocks
            if q_lens[s]:
                pos = np.arange(first_pos[s], ctx_len[s])
                pages = np.asarray(e.seq.blocks[gi], dtype=np.int64)[pos // bs]
                slots[starts[s]:starts[s] + q_lens[s]] = pages * bs + pos % bs
        names += [f"tables{gi}", f"slots{gi}"]
        arrays += [tables, slots]
    decode_ctx = [int(c) for c, q in zip(ctx_len, q_lens) if q == 1]
    host = {"q_start": starts, "q_len": q_len, "ctx_len": ctx_len, "positions": positions, "token_ids": token_ids,
            "state_slots": state_slots, "seq_of_token": seq_of_token, "first_pos": first_pos}
    return StepArrays(names, arrays, lists, T, len(entries), len(rows), max(q_lens, default=0), max(decode_ctx, default=0),
                      max((int(c) for c in ctx_len), default=0), ops.mean_tile_walk(q_lens, ctx_len), host)


def context_from(step: StepArrays, dev: list, n_groups: int, workspace: Workspace, act_dtype, attention_kind: int = 0,
                 max_decode_ctx: int | None = None, max_ctx: int | None = None) -> StepContext:
    """The step's context over the device copies `dev` of `step.arrays` (same order)."""
    ctx = StepContext(workspace, act_dtype, attention_kind)
    by_name = dict(zip(step.names, dev))
    ctx.token_ids, ctx.positions, ctx.q_start = by_name["token_ids"], by_name["positions"], by_name["q_start"]
    ctx.q_len, ctx.ctx_len, ctx.logit_rows = by_name["q_len"], by_name["ctx_len"], by_name["logit_rows"]
    ctx.state_slots, ctx.seq_of_token = by_name["state_slots"], by_name["seq_of_token"]
    ctx.extra = {name[2:]: tensor for name, tensor in by_name.items() if name.startswith("x:")}
    on_device = {name: (by_name[name], len(step.lists[name])) for name in step.lists}
    ctx.attention = ops.AttentionBatch(ctx.q_start, ctx.q_len, ctx.ctx_len, step.n_seqs, on_device,
                                       step.max_decode_ctx if max_decode_ctx is None else max_decode_ctx,
                                       step.max_ctx if max_ctx is None else max_ctx, step.mean_walk)
    ctx.group_tables = [by_name[f"tables{g}"] for g in range(n_groups)]
    ctx.group_slots = [by_name[f"slots{g}"] for g in range(n_groups)]
    ctx.n_tokens, ctx.n_seqs, ctx.n_logits = step.n_tokens, step.n_seqs, step.n_logits
    ctx.max_q_len = step.max_q_len
    ctx.host = step.host
    return ctx


def build_context(entries: list[StepEntry], cache, stager: DescriptorStager, workspace: Workspace, act_dtype,
                  attention_kind: int = 0) -> StepContext:
    """Lay the entries out flat and stage every array the kernels need, in one copy to the device."""
    step = step_arrays(entries, cache)
    return context_from(step, stager.upload(step.arrays), len(cache.groups), workspace, act_dtype, attention_kind)
