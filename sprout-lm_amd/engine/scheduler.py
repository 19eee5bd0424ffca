"""Continuous batching with chunked prefill: which requests run which tokens in the next step.

Reference: Engine (src/engine.ts:42-241).  The policy is the reference's: first come first admitted
up to max_sequences; decoding requests before prefilling ones, then by arrival; a token budget per
step; prompts cut into portions; when pages run out the youngest younger request is preempted
(its pages are given back, its tokens are kept and its cache is rebuilt later), and a request with
no younger one to preempt steps back itself.  Unlike the reference, which reserves pages token by
token while it computes, all pages of a step are settled here before anything is launched, so a
request that is preempted while the step is planned brings no tokens to that step.

The scheduler decides and keeps the books; it launches nothing.  `plan()` returns the work of the
next step, the caller runs it and reports the sampled tokens to `complete()`.  While a step of decoded
tokens runs, `plan_ahead()` may already settle the step after it, so that the host's work for one step
overlaps the GPU's work for the other (no counterpart in the reference, whose steps are synchronous).
"""
from __future__ import annotations

from dataclasses import dataclass, field

from ..cache.manager import CacheManager, SequenceCache
from ..config.engine_options import EngineOptions
from ..sampling.params import SamplingParams


class RequestRefused(ValueError):
    """A request that can never run: its id, its tokens or its length do not fit this engine."""


@dataclass(frozen=True)
class Limits:
    """What a request is measured against when it arrives."""

    vocab_size: int
    max_context: int      # positions the model has
    pool_tokens: int      # token slots of the whole cache pool


@dataclass(frozen=True)
class Event:
    """Something that happened to a request in a scheduling round.  Reports and traces carry `to_dict()`."""

    tick: int
    id: str
    kind: str             # queued | admitted | token | finished | cancelled | preempted
    detail: str
    extra: tuple = ()     # (key, value) pairs of the kind's own fields: token and index, finish_reason

    def to_dict(self) -> dict:
        return {"tick": self.tick, "id": self.id, "type": self.kind, "detail": self.detail, **dict(self.extra)}


@dataclass
class Request:
    id: str
    order: int
    prompt: list
    max_new_tokens: int
    params: SamplingParams
    output: list = field(default_factory=list)
    status: str = "waiting"            # waiting | running | finished | cancelled
    seq: SequenceCache | None = None
    prefix_hits: int = 0
    finish_reason: str | None = None   # eos | length
    preemptions: int = 0

    @classmethod
    def checked(cls, id, order: int, prompt, max_new_tokens, params: SamplingParams, limits: Limits, known_ids) -> "Request":
        """A new request, or RequestRefused saying what is wrong with it.  What is checked is what the reference
        checks when a request arrives (src/engine.ts:74-85): the id, the token ids, the number of new tokens, and
        that the request could run at all: the last token it samples is never fed back, so it needs one cache slot
        less than it has tokens."""
        if not isinstance(id, str) or id == "" or id in known_ids:
            raise RequestRefused(f"A request needs an id of its own: {id!r} is empty, no string, or already in use.")
        tokens = list(prompt)
        if not tokens:
            raise RequestRefused(f"Request {id!r} brings no prompt: at least one token id in [0, {limits.vocab_size}) is needed.")
        for place, token in enumerate(tokens):
            if isinstance(token, bool) or not isinstance(token, int) or not 0 <= token < limits.vocab_size:
                raise RequestRefused(f"Request {id!r}: prompt[{place}] = {token!r} is no token id in [0, {limits.vocab_size}).")
        if isinstance(max_new_tokens, bool) or not isinstance(max_new_tokens, int) or max_new_tokens < 1:
            raise RequestRefused(f"Request {id!r}: max_new_tokens must be a positive integer, got {max_new_tokens!r}.")
        slots = len(tokens) + max_new_tokens - 1
        if slots > limits.max_context:
            raise RequestRefused(f"Request {id!r}: {len(tokens)} prompt tokens and {max_new_tokens} new ones need "
                                 f"{slots} positions, the model has {limits.max_context}.")
        if slots > limits.pool_tokens:
            raise RequestRefused(f"Request {id!r}: {slots} cache slots are more than the whole pool holds "
                                 f"({limits.pool_tokens} = num_blocks x block_size), even with nothing else running.")
        return cls(id, order, tokens, max_new_tokens, params)

    def history(self) -> list:
        return self.prompt + self.output

    def history_length(self) -> int:
        return len(self.prompt) + len(self.output)

    def history_slice(self, start: int, stop: int) -> list:
        """history()[start:stop] without building the whole history."""
        n = len(self.prompt)
        if stop <= n:
            return self.prompt[start:stop]
        if start >= n:
            return self.output[start - n:stop - n]
        return self.prompt[start:] + self.output[:stop - n]


@dataclass
class Work:
    """One request's share of a step."""

    request: Request
    phase: str          # prefill | decode | recompute
    start: int          # position of the first token ("from" in the reference's report)
    tokens: list
    samples: bool       # the last token of the history is in this share: a new token is sampled

    def report(self) -> dict:
        return {"id": self.request.id, "phase": self.phase, "from": self.start, "tokens": len(self.tokens),
                "block_table": [list(b) for b in self.request.seq.blocks] if self.request.seq else []}


class Scheduler:
    def __init__(self, cache: CacheManager, options: EngineOptions, vocab_size: int, max_context: int,
                 eos_token_ids=()):
        self.cache, self.options = cache, options
        self.vocab_size, self.max_context = vocab_size, max_context
        self.eos_token_ids = tuple(eos_token_ids)
        self.limits = Limits(vocab_size, max_context, options.num_blocks * options.block_size)
        self.requests: dict[str, Request] = {}
        self.active: dict[str, Request] = {}
        self.waiting: list[str] = []
        self.trace: list[dict] = []
        self.tick = 0
        self._arrivals = 0
        self._step_events: list[dict] | None = None
        self.stats = {"preemptions": 0, "recomputed_tokens": 0, "prefix_hit_tokens": 0}

    # ------------------------------------------------------------------ requests
    def add(self, id: str, prompt, max_new_tokens: int, params: SamplingParams | None = None) -> None:
        """Take a request into the waiting line (first come, first admitted), or raise RequestRefused."""
        request = Request.checked(id, self._arrivals, prompt, max_new_tokens, params or SamplingParams(), self.limits,
                                  self.requests)
        self._arrivals += 1
        self.requests[request.id] = request
        self.waiting.append(request.id)
        self._note(request, "queued", f"waits with {len(request.prompt)} prompt tokens for up to {max_new_tokens} new ones")

    @property
    def pending(self) -> bool:
        return bool(self.active or self.waiting)

    def _alive(self, id: str) -> Request | None:
        """The request if it still waits or runs."""
        request = self.requests.get(id)
        return request if request is not None and request.status in ("waiting", "running") else None

    def forget(self, id: str) -> bool:
        """Drop the record of a request that has ended; False for one that is unknown or still alive."""
        if id not in self.requests or self._alive(id) is not None:
            return False
        del self.requests[id]
        return True

    def cancel(self, id: str) -> bool:
        """End a waiting or running request now.  Its pages go back to the pool at once (pages it shares with
        the prefix cache or with other requests stay with those); False if there was nothing to end."""
        request = self._alive(id)
        if request is None:
            return False
        held = sum(len(b) for b in request.seq.blocks) if request.seq else 0
        self._leave(request, "cancelled")
        self._note(request, "cancelled", f"stopped after {len(request.output)} tokens; {held} page references given back")
        return True

    def result(self, id: str) -> dict:
        """Where a request stands (reference: Engine.result, src/engine.ts:111-124, plus `preemptions`)."""
        if id not in self.requests:
            raise KeyError(f"No request {id!r} is known to the engine (finished requests stay until `forget`).")
        request = self.requests[id]
        seq = request.seq
        return {"id": id, "status": request.status, "output": list(request.output),
                "finish_reason": request.finish_reason,
                "computed_tokens": seq.length if seq else 0,
                "block_table": list(seq.blocks[0]) if seq and seq.blocks else [],
                "prefix_hits": request.prefix_hits, "preemptions": request.preemptions}

    # ------------------------------------------------------------------ one step
    def plan(self) -> list[Work]:
        """Choose the next step's work and reserve every page it needs (src/engine.ts:137-189)."""
        self.tick += 1
        self._step_events = []
        self._admit()
        budget = self.options.max_batch_tokens
        planned: dict[str, Work] = {}
        phases = {r.id: self._phase(r) for r in self.active.values()}
        batch = sorted(self.active.values(), key=lambda r: (phases[r.id] != "decode", r.order))
        for request in batch:
            if budget <= 0:
                break
            if request.status != "running":
                continue   # an older request preempted it while this step was planned
            total = request.history_length()
            phase = phases[request.id]
            start = request.seq.length
            remaining = total - start - (phase == "recompute")
            count = min(budget, 1 if phase == "decode" else self.options.prefill_chunk_size, remaining)
            multiple = self.options.step_token_multiple
            closes_step = False
            if multiple > 1 and phase != "decode" and count < remaining:
                # a portion that carries the step over a whole multiple is cut back to it and closes the step
                # (a portion that ends its prompt is left alone: the request's first token is not held back)
                used = sum(len(w.tokens) for w in planned.values())
                aligned = (used + count) // multiple * multiple - used
                if 0 < aligned < count:
                    count, closes_step = aligned, True
            if count <= 0:
                continue
            ok, refund = self._reserve(request, start + count, planned)
            budget += refund
            if not ok:
                continue      # the step goes on with its whole budget: nothing was cut for a portion that is not in it
            tokens = request.history_slice(start, start + count)
            planned[request.id] = Work(request, phase, start, tokens, samples=start + count == total)
            budget = 0 if closes_step else budget - count
        return [planned[r.id] for r in batch if r.id in planned]

    def plan_ahead(self, running: list[Work]) -> list[Work] | None:
        """The step after `running`, planned while that step is still being computed.

        Possible only where the next step can be foreseen without the tokens on their way: `running` is a
        step of single decoded tokens of every active request, nobody waits for admission, and every
        request that goes on has a page for one more token (nothing is preempted on a guess).  A request
        that will reach its token limit is left out; one that turns out to have stopped at an end token is
        not known yet and is included: its share of the step is computed in vain and ignored by
        `complete`.  The tokens of the returned work are [None]: they are not known on the host.
        Returns None when the caller should wait for the running step and `plan()` as usual.
        """
        if self.waiting or not running:
            return None
        if any(w.phase != "decode" or not w.samples for w in running):
            return None
        alive = [w.request for w in running if w.request.status == "running"]
        if len(alive) != len(self.active) or any(r.id not in self.active for r in alive):
            return None
        if any(r.seq.length != r.history_length() for r in alive):
            return None        # `running` has not been launched: its tokens are not in the cache yet
        ahead = [r for r in alive if len(r.output) + 1 < r.max_new_tokens]
        if not ahead:
            return None
        for r in ahead:
            if not self.cache.reserve(r.seq, r.seq.length + 1):
                return None
        return [Work(r, "decode", r.seq.length, [None], samples=True) for r in ahead]

    def begin_ahead(self) -> None:
        """A step planned by `plan_ahead` becomes the current one (what `plan()` does besides choosing)."""
        self.tick += 1
        self._step_events = []

    def complete(self, work: list[Work], sampled: dict[str, int]) -> list[dict]:
        """Book a finished step: lengths have advanced; `sampled` maps request id -> new token."""
        for w in work:
            request = w.request
            if request.status != "running":
                continue   # cancelled between plan and completion
            seq = request.seq
            if w.phase == "recompute":
                self.stats["recomputed_tokens"] += len(w.tokens)
            if self.cache.prefix_caching:
                bs = self.cache.block_size
                limit = min(seq.length, len(request.prompt))
                for boundary in range((w.start // bs + 1) * bs, limit + 1, bs):
                    self.cache.publish(request.prompt, seq, boundary)
            if not w.samples:
                continue
            token = sampled[request.id]
            if isinstance(token, bool) or not isinstance(token, int) or token < 0 or token >= self.vocab_size:
                raise RuntimeError("Runner returned invalid sampled token.")
            request.output.append(token)
            self._note(request, "token", f"token {token}", token=token, index=len(request.output) - 1)
            stops = request.params.stop_token_ids if request.params.stop_token_ids is not None else self.eos_token_ids
            eos = token in stops and not request.params.ignore_eos
            if eos or len(request.output) == request.max_new_tokens:
                request.finish_reason = "eos" if eos else "length"
                self._leave(request, "finished")
                self._note(request, "finished", f"{len(request.output)} tokens, ended by "
                           + ("a stop token" if eos else "its length limit"), finish_reason=request.finish_reason)
        events, self._step_events = self._step_events or [], None
        return events

    def fail_all(self, reason: str) -> None:
        """A step failed: every request ends and every page comes back (reference: src/service.ts:222-231)."""
        for request in list(self.requests.values()):
            if request.status in ("waiting", "running"):
                self._leave(request, "cancelled")
                self._note(request, "cancelled", f"engine_error: {reason}")
        self.cache.clear_prefixes()

    # ------------------------------------------------------------------ internals
    def _phase(self, request: Request) -> str:
        if not request.output:
            return "prefill"
        return "recompute" if request.seq.length < len(request.prompt) + len(request.output) - 1 else "decode"

    def _admit(self) -> None:
        """Waiting requests start in arrival order while a sequence slot is free.  A request that was preempted
        comes back with its output: whatever of its prompt still lies in cached pages is found again, the rest of
        its history is computed again (reference: src/engine.ts:197-207)."""
        while self.waiting and len(self.active) < self.options.max_sequences:
            request = self.requests[self.waiting.pop(0)]
            if self.options.prefix_caching:
                request.seq = self.cache.reuse_prefix(request.history())
            else:
                request.seq = self.cache.create()
            found = request.seq.length
            request.prefix_hits += found
            self.stats["prefix_hit_tokens"] += found
            request.status = "running"
            self.active[request.id] = request
            self._note(request, "admitted", f"{found} of {request.history_length()} tokens found in cached pages "
                       f"{[list(b) for b in request.seq.blocks]}" if found else f"starts with an empty cache")

    def _reserve(self, request: Request, new_length: int, planned: dict) -> tuple[bool, int]:
        """Pages for `request` up to `new_length`; preempts younger requests, else the request itself.

        Returns (reserved, token budget given back by preempted requests that were already planned).
        Older requests are never preempted by younger ones, so a crowded pool still makes progress
        (src/engine.ts:209-222).
        """
        refund = 0
        while not self.cache.reserve(request.seq, new_length):
            younger = [r for r in self.active.values() if r.order > request.order]
            if not younger:
                self._preempt(request)
                return False, refund
            victim = max(younger, key=lambda r: r.order)
            dropped = planned.pop(victim.id, None)
            if dropped is not None:
                refund += len(dropped.tokens)
            self._preempt(victim)
        return True, refund

    def _preempt(self, request: Request) -> None:
        """Back to the end of the waiting line with nothing but its tokens (src/engine.ts:224-231)."""
        self._leave(request, "waiting")
        request.preemptions += 1
        self.stats["preemptions"] += 1
        self.waiting.append(request.id)
        self._note(request, "preempted", f"pages given up for an older request; its {len(request.output)} tokens are "
                   f"kept and the cache is computed again after readmission")

    def _leave(self, request: Request, status: str) -> None:
        """The request stops running or waiting: its cache goes back to the pool, the books forget it."""
        if request.seq is not None:
            request.seq.release()
            request.seq = None
        request.status = status
        self.active.pop(request.id, None)
        if request.id in self.waiting:
            self.waiting.remove(request.id)

    def _note(self, request: Request, kind: str, detail: str, **extra) -> None:
        event = Event(self.tick, request.id, kind, detail, tuple(extra.items())).to_dict()
        if self.options.record_trace:
            self.trace.append(event)
        if self._step_events is not None:
            self._step_events.append(event)
