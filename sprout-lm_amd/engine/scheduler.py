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
        self.requests: dict[str, Request] = {}
        self.active: dict[str, Request] = {}
        self.waiting: list[str] = []
        self.trace: list[dict] = []
        self.tick = 0
        self._next_order = 0
        self._step_events: list[dict] | None = None
        self.stats = {"preemptions": 0, "recomputed_tokens": 0, "prefix_hit_tokens": 0}

    # ------------------------------------------------------------------ requests
    def add(self, id: str, prompt, max_new_tokens: int, params: SamplingParams | None = None) -> None:
        """Reference: Engine.add, src/engine.ts:74-93 (same checks, same order)."""
        if not isinstance(id, str) or not id or id in self.requests:
            raise ValueError("Request ID must be nonempty and unique.")
        prompt = list(prompt)
        if not prompt or any(isinstance(t, bool) or not isinstance(t, int) or t < 0 or t >= self.vocab_size for t in prompt):
            raise ValueError("Prompt must contain valid token IDs.")
        if isinstance(max_new_tokens, bool) or not isinstance(max_new_tokens, int) or max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be a positive integer.")
        # the last sampled token is never fed back, so it needs no cache slot
        slots = len(prompt) + max_new_tokens - 1
        if slots > self.max_context:
            raise ValueError("Request exceeds the model context limit.")
        if slots > self.options.num_blocks * self.options.block_size:
            raise ValueError("Request cannot fit alone in the KV pool. Increase num_blocks or shorten it.")
        request = Request(id, self._next_order, prompt, max_new_tokens, params or SamplingParams())
        self._next_order += 1
        self.requests[id] = request
        self.waiting.append(id)
        self._emit("queued", request, f"{len(prompt)} prompt tokens")

    @property
    def pending(self) -> bool:
        return bool(self.active or self.waiting)

    def forget(self, id: str) -> bool:
        request = self.requests.get(id)
        if request is None or request.status in ("waiting", "running"):
            return False
        del self.requests[id]
        return True

    def cancel(self, id: str) -> bool:
        request = self.requests.get(id)
        if request is None or request.status in ("finished", "cancelled"):
            return False
        self._drop_cache(request)
        request.status = "cancelled"
        self.active.pop(id, None)
        self.waiting = [w for w in self.waiting if w != id]
        self._emit("cancelled", request, "Released live KV references")
        return True

    def result(self, id: str) -> dict:
        request = self.requests.get(id)
        if request is None:
            raise KeyError(f"Unknown request: {id}")
        return {"id": id, "status": request.status, "output": list(request.output),
                "finish_reason": request.finish_reason,
                "computed_tokens": request.seq.length if request.seq else 0,
                "block_table": list(request.seq.blocks[0]) if request.seq and request.seq.blocks else [],
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
            if multiple > 1 and phase != "decode" and count < remaining:
                # a portion that carries the step over a whole multiple is cut back to it and closes the step
                # (a portion that ends its prompt is left alone: the request's first token is not held back)
                used = sum(len(w.tokens) for w in planned.values())
                aligned = (used + count) // multiple * multiple - used
                if 0 < aligned < count:
                    count = aligned
                    budget = count
            if count <= 0:
                continue
            ok, refund = self._reserve(request, start + count, planned)
            budget += refund
            if not ok:
                continue
            tokens = request.history_slice(start, start + count)
            planned[request.id] = Work(request, phase, start, tokens, samples=start + count == total)
            budget -= count
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
            self._emit("token", request, str(token), token=token, index=len(request.output) - 1)
            stops = request.params.stop_token_ids if request.params.stop_token_ids is not None else self.eos_token_ids
            eos = token in stops and not request.params.ignore_eos
            if eos or len(request.output) == request.max_new_tokens:
                request.finish_reason = "eos" if eos else "length"
                request.status = "finished"
                self._drop_cache(request)
                del self.active[request.id]
                self._emit("finished", request, f"{len(request.output)} output tokens",
                           finish_reason=request.finish_reason)
        events, self._step_events = self._step_events or [], None
        return events

    def fail_all(self, reason: str) -> None:
        """A step failed: every request ends and every page comes back (reference: src/service.ts:222-231)."""
        for request in list(self.requests.values()):
            if request.status in ("waiting", "running"):
                self._drop_cache(request)
                request.status = "cancelled"
                self._emit("cancelled", request, f"engine_error: {reason}")
        self.active.clear()
        self.waiting.clear()
        self.cache.clear_prefixes()

    # ------------------------------------------------------------------ internals
    def _phase(self, request: Request) -> str:
        if not request.output:
            return "prefill"
        return "recompute" if request.seq.length < len(request.prompt) + len(request.output) - 1 else "decode"

    def _admit(self) -> None:
        while len(self.active) < self.options.max_sequences and self.waiting:
            request = self.requests[self.waiting.pop(0)]
            history = request.history()
            request.seq = self.cache.reuse_prefix(history) if self.options.prefix_caching else self.cache.create()
            request.prefix_hits += request.seq.length
            self.stats["prefix_hit_tokens"] += request.seq.length
            request.status = "running"
            self.active[request.id] = request
            self._emit("admitted", request, f"Reused {request.seq.length} prefix tokens; pages {request.seq.blocks}")

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
        self._drop_cache(request)
        request.status = "waiting"
        request.preemptions += 1
        self.stats["preemptions"] += 1
        del self.active[request.id]
        self.waiting.append(request.id)
        self._emit("preempted", request, "Keep output tokens; rebuild missing KV after readmission")

    def _drop_cache(self, request: Request) -> None:
        if request.seq is not None:
            request.seq.release()
            request.seq = None

    def _emit(self, type: str, request: Request, detail: str, **extra) -> None:
        event = {"tick": self.tick, "id": request.id, "type": type, "detail": detail, **extra}
        if self.options.record_trace:
            self.trace.append(event)
        if self._step_events is not None:
            self._step_events.append(event)
