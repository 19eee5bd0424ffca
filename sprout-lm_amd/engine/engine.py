"""The serving engine: request table, scheduler, step function and sampler in one loop.

Reference: Engine (src/engine.ts:42-241) for add/step/cancel/forget/result/pending, and
GenerationService.generate (src/service.ts:144-173) for `stream`.
"""
from __future__ import annotations

import itertools
from dataclasses import asdict

from ..config.engine_options import EngineOptions
from ..sampling.params import SamplingParams
from .batch import StepEntry
from .scheduler import Scheduler, Work


class StepReport:
    """What one scheduling iteration did (reference: src/engine.ts:27-33, :189)."""

    def __init__(self, tick, work, events, cache, replayed=False, launched_ahead=False):
        self.tick, self.work, self.events = tick, work, events
        # beyond the reference's report: the step ran as a replay of a recorded graph; it had been launched
        # before the step before it was read back
        self.replayed, self.launched_ahead = replayed, launched_ahead
        self._cache = cache
        self._memory = None

    @property
    def memory(self) -> dict:
        if self._memory is None:
            self._memory = self._cache.snapshot()
        return self._memory

    def to_dict(self) -> dict:
        return {"tick": self.tick, "work": self.work, "events": self.events, "memory": self.memory,
                "replayed": self.replayed, "launched_ahead": self.launched_ahead}


class Engine:
    def __init__(self, model, options: EngineOptions | None = None, sampler=None, **overrides):
        """`model` is a ModelRunner (or anything with its `cache`, `step`, sizes and stop ids).

        The cache geometry in `options` must be the one the model's cache was made with.
        """
        cache = model.cache
        base = asdict(options) if options is not None else {}
        base.update(overrides)
        base.setdefault("block_size", cache.block_size)
        base.setdefault("num_blocks", cache.num_blocks)
        base.setdefault("max_sequences", cache.max_sequences)
        self.options = EngineOptions(**base)
        if (self.options.block_size, self.options.num_blocks) != (cache.block_size, cache.num_blocks) \
                or self.options.max_sequences > cache.max_sequences:
            raise ValueError("Engine options and the model's cache differ in block_size, num_blocks or max_sequences.")
        self.model, self.cache = model, cache
        self.sampler = sampler     # None: the model samples on the device (`step_and_sample`)
        self.scheduler = Scheduler(cache, self.options, model.vocab_size, model.max_positions, model.stop_token_ids)
        self._auto_ids = itertools.count()
        self._ahead = None      # (work, handle) of a step launched before its predecessor was read back

    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", options: EngineOptions | None = None, **overrides) -> "Engine":
        from .runner import ModelRunner
        options = EngineOptions(**{**(asdict(options) if options else {}), **overrides})
        runner = ModelRunner.from_folder(folder, dtype, block_size=options.block_size, num_blocks=options.num_blocks,
                                         max_sequences=options.max_sequences, prefix_caching=options.prefix_caching,
                                         strict_tensors=options.strict_tensors,
                                         weight_limit_mib=options.weight_limit_mib, reserve_mib=options.reserve_mib)
        return cls(runner, options)

    @classmethod
    def from_config(cls, config, seed: int = 0, dtype="bfloat16", options: EngineOptions | None = None,
                    **overrides) -> "Engine":
        from .runner import ModelRunner
        options = EngineOptions(**{**(asdict(options) if options else {}), **overrides})
        runner = ModelRunner.from_config(config, seed, dtype, block_size=options.block_size,
                                         num_blocks=options.num_blocks, max_sequences=options.max_sequences,
                                         prefix_caching=options.prefix_caching,
                                         weight_limit_mib=options.weight_limit_mib, reserve_mib=options.reserve_mib)
        return cls(runner, options)

    # ------------------------------------------------------------------ the reference's surface
    def add(self, id: str | None = None, prompt=(), max_new_tokens: int = 16, temperature: float = 0.0, seed: int = 0,
            stop_token_ids=None, ignore_eos: bool = False) -> str:
        if id is None:
            id = f"request-{next(self._auto_ids)}"
        params = SamplingParams(temperature, seed, None if stop_token_ids is None else tuple(stop_token_ids), ignore_eos)
        self.scheduler.add(id, prompt, max_new_tokens, params)
        return id

    @property
    def pending(self) -> bool:
        return self.scheduler.pending

    @property
    def trace(self) -> list:
        return self.scheduler.trace

    def cancel(self, id: str) -> bool:
        return self.scheduler.cancel(id)

    def forget(self, id: str) -> bool:
        return self.scheduler.forget(id)

    def result(self, id: str) -> dict:
        return self.scheduler.result(id)

    def step(self) -> StepReport:
        """One scheduling iteration: plan, run the batch, sample, book (src/engine.ts:127-189).

        A step of decoded tokens is launched and, before its tokens are read back, the step after it is
        planned and launched as well where the scheduler can foresee it (`plan_ahead`): the host then
        plans one step while the GPU computes the other.  That step is booked by the next call.
        """
        ahead, self._ahead = self._ahead, None
        if ahead is not None and not any(w.request.status == "running" for w in ahead[0]):
            self._discard(ahead)    # every request of it has ended meanwhile: nothing to book
            ahead = None
        if ahead is not None:
            work, pending = ahead
            self.scheduler.begin_ahead()
        else:
            work, pending = self.scheduler.plan(), None
        sampled: dict[str, int] = {}
        reports = []
        if work:
            sampling = [w for w in work if w.samples]
            try:
                if pending is None:
                    entries = [StepEntry(w.request.seq, w.tokens, [len(w.tokens) - 1] if w.samples else []) for w in work]
                    params = [w.request.params for w in sampling]
                    counters = [len(w.request.output) for w in sampling]
                    launch = getattr(self.model, "launch_decode", None) if self.sampler is None else None
                    if launch is not None:
                        pending = launch(entries, params, counters)
                if pending is not None:
                    self._launch_ahead(work, pending)
                    tokens = self.model.finish_decode(pending)
                elif self.sampler is None:
                    tokens = self.model.step_and_sample(entries, params, counters)
                else:
                    tokens = self.sampler.sample(self.model.step(entries), params, counters)
            except Exception as error:
                if self._ahead is not None:
                    self._discard(self._ahead)
                    self._ahead = None
                self.scheduler.fail_all(str(error))
                raise
            sampled = {w.request.id: t for w, t in zip(sampling, tokens)}
            reports = [w.report() for w in work]
        events = self.scheduler.complete(work, sampled)
        return StepReport(self.scheduler.tick, reports, events, self.cache, replayed=pending is not None,
                          launched_ahead=ahead is not None)

    @staticmethod
    def _discard(ahead) -> None:
        """Wait for a launched step whose result nobody wants: what it reads and writes (cache pages, the
        recorded graph and its buffers) must not be given back or destroyed under it."""
        try:
            ahead[1].result()
        except Exception:
            pass

    def _launch_ahead(self, work, pending) -> None:
        """Plan and launch the step after `work` (which runs as `pending`) if it can be foreseen."""
        if not self.options.decode_lookahead:
            return
        following = self.scheduler.plan_ahead(work)
        if not following:
            return
        row = {w.request.id: i for i, w in enumerate(work)}
        entries = [StepEntry(w.request.seq, [None], [0]) for w in following]
        sources = [row[w.request.id] for w in following]
        params = [w.request.params for w in following]
        counters = [len(w.request.output) + 1 for w in following]     # the running step's token comes first
        launched = self.model.launch_decode(entries, params, counters, feed=(pending, sources))
        if launched is not None:
            self._ahead = (following, launched)

    # ------------------------------------------------------------------ conveniences
    def generate(self, prompts, max_new_tokens: int = 16, temperature: float = 0.0, seed: int = 0,
                 ignore_eos: bool = False, step_limit: int = 1_000_000) -> list[list[int]]:
        """Run `prompts` (lists of token ids) to the end; returns their output token ids in order."""
        ids = [self.add(None, p, max_new_tokens, temperature, seed + i, None, ignore_eos) for i, p in enumerate(prompts)]
        steps = 0
        while any(self.scheduler.requests[i].status in ("waiting", "running") for i in ids):
            steps += 1
            if steps > step_limit:
                raise RuntimeError("The scheduler made no progress.")
            self.step()
        outputs = [self.result(i)["output"] for i in ids]
        for i in ids:
            self.forget(i)
        return outputs

    def stream(self, prompt, max_new_tokens: int = 16, id: str | None = None, **sampling):
        """Events of one request as they happen: queued, token ..., finished (with usage).

        Other queued requests advance in the same steps.  Reference: src/service.ts:144-173.
        """
        id = self.add(id, prompt, max_new_tokens, **sampling)
        yield {"id": id, "type": "queued"}
        while self.scheduler.requests[id].status in ("waiting", "running"):
            for event in self.step().events:
                if event["id"] != id:
                    continue
                if event["type"] == "token":
                    yield {"id": id, "type": "token", "token": event["token"], "index": event["index"]}
        request = self.scheduler.requests[id]
        usage = {"prompt_tokens": len(request.prompt), "completion_tokens": len(request.output)}
        if request.status == "finished":
            yield {"id": id, "type": "finished", "finish_reason": request.finish_reason, "usage": usage}
        else:
            yield {"id": id, "type": "cancelled", "usage": usage}
        self.forget(id)

    def stats(self) -> dict:
        return {**self.scheduler.stats, "tick": self.scheduler.tick, "free_pages": self.cache.free_pages(),
                "evictions": self.cache.evictions}

    def close(self) -> None:
        if self._ahead is not None:
            self._discard(self._ahead)
            self._ahead = None
        self.scheduler.fail_all("closed")

    def __del__(self):
        ahead = getattr(self, "_ahead", None)
        if ahead is not None:
            self._discard(ahead)
