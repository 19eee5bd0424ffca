"""The scheduler's decisions, on the CPU with a stand-in model (reference: test/engine.test.ts, test/qwen.test.ts:48-117)."""
import pytest

from sprout_lm_amd.engine import Engine
from tests.fake_model import ArgmaxSampler, FakeRunner


def make(block_size=4, num_blocks=64, max_sequences=4, prefix_caching=True, eos=(), **options):
    runner = FakeRunner(block_size, num_blocks, max_sequences, prefix_caching, eos)
    options.setdefault("max_batch_tokens", 8)
    options.setdefault("prefill_chunk_size", 4)
    options.setdefault("record_trace", True)
    return Engine(runner, sampler=ArgmaxSampler(), prefix_caching=prefix_caching, **options)


def drain(engine, limit=2000):
    reports = []
    while engine.pending:
        assert len(reports) < limit, "scheduler must make progress"
        report = engine.step()
        assert sum(w["tokens"] for w in report.work) <= engine.options.max_batch_tokens
        assert all(p["refs"] >= 0 and p["active_refs"] >= 0 for p in report.memory["pages"])
        reports.append(report)
    return reports


def prompt(text):
    return [ord(c) % 50 for c in text]


def test_late_request_joins_and_decode_mixes_with_chunked_prefill():
    engine = make(max_batch_tokens=6, prefill_chunk_size=3, max_sequences=3)
    prompts = [prompt("a"), prompt("longer prompt"), prompt("late")]
    engine.add("A", prompts[0], 6)
    engine.add("B", prompts[1], 3)
    engine.step()
    engine.add("C", prompts[2], 2)
    reports = drain(engine)
    assert any({w["phase"] for w in r.work} >= {"decode", "prefill"} for r in reports)
    for rid, p, n in zip("ABC", prompts, (6, 3, 2)):
        result = engine.result(rid)
        assert result["status"] == "finished" and result["finish_reason"] == "length"
        assert result["output"] == engine.model.greedy(p, n)
    kinds = [(e["id"], e["type"]) for e in engine.trace]
    assert kinds.index(("C", "admitted")) < kinds.index(("B", "finished"))
    assert max(engine.model.steps) <= 6


def test_decode_goes_first_and_budget_cuts_prompts():
    engine = make(max_batch_tokens=5, prefill_chunk_size=4, max_sequences=3)
    engine.add("A", prompt("ab"), 4)
    engine.step()                                  # A prefilled (2 tokens) and sampled
    engine.add("B", prompt("0123456789"), 1)
    report = engine.step()
    assert [(w["id"], w["phase"], w["from"], w["tokens"]) for w in report.work] == [("A", "decode", 2, 1), ("B", "prefill", 0, 4)]
    report = engine.step()
    assert [(w["id"], w["from"], w["tokens"]) for w in report.work] == [("A", 3, 1), ("B", 4, 4)]
    drain(engine)


def test_a_step_is_cut_back_to_a_whole_multiple_of_tokens():
    """step_token_multiple: the portion that carries a step over a multiple is shortened and closes the step;
    a portion that ends its prompt is left alone; outputs do not change."""
    texts = {"A": "ab", "B": "0123456789abcdefghijklm", "C": "zyxwvutsr"}
    outputs = {}
    for multiple in (1, 4):
        engine = make(max_batch_tokens=16, prefill_chunk_size=6, max_sequences=3, step_token_multiple=multiple,
                      prefix_caching=False)
        engine.add("A", prompt(texts["A"]), 6)
        engine.step()                                  # A prefilled (2 tokens) and sampled
        engine.add("B", prompt(texts["B"]), 2)
        engine.add("C", prompt(texts["C"]), 2)
        report = engine.step()
        work = [(w["id"], w["phase"], w["tokens"]) for w in report.work]
        if multiple == 1:
            assert work == [("A", "decode", 1), ("B", "prefill", 6), ("C", "prefill", 6)]
        else:                                          # 1 + 6 = 7 crosses 4: B is cut to 3 and closes the step
            assert work == [("A", "decode", 1), ("B", "prefill", 3)]
        reports = [report] + drain(engine)
        if multiple > 1:
            for r in reports:                          # every other step: a whole multiple, or a prompt ends in it
                total = sum(w["tokens"] for w in r.work)
                ends = any(w["phase"] == "prefill" and w["from"] + w["tokens"] == len(texts[w["id"]]) for w in r.work)
                assert total <= multiple or total % multiple == 0 or ends, (total, r.work)
        outputs[multiple] = {rid: engine.result(rid)["output"] for rid in "ABC"}
        for rid, n in (("A", 6), ("B", 2), ("C", 2)):
            assert outputs[multiple][rid] == engine.model.greedy(prompt(texts[rid]), n)
    assert outputs[1] == outputs[4]


def test_prefix_sharing_reuses_pages_and_recomputes_the_last_prompt_token():
    engine = make(block_size=2, prefill_chunk_size=8)
    p = prompt("abcd")                             # exactly two full pages
    engine.add("A", p, 4)
    engine.step()
    a_pages = engine.result("A")["block_table"]
    engine.add("B", p, 4)
    report = engine.step()
    assert engine.result("B")["prefix_hits"] == 2
    assert engine.result("B")["block_table"][0] == a_pages[0]
    assert report.memory["pages"][a_pages[0]]["active_refs"] == 2
    drain(engine)
    assert engine.result("A")["output"] == engine.result("B")["output"] == engine.model.greedy(p, 4)
    assert all(page["active_refs"] == 0 for page in engine.cache.snapshot()["pages"])
    engine.cache.clear_prefixes()
    assert engine.cache.free_pages() == [engine.options.num_blocks]


def test_same_suffix_under_another_context_does_not_hit():
    engine = make(block_size=2, prefill_chunk_size=8)
    engine.add("A", [1, 2, 3, 4, 5], 1)
    drain(engine)
    engine.add("B", [9, 8, 3, 4, 5], 1)
    drain(engine)
    assert engine.result("B")["prefix_hits"] == 0
    assert engine.result("B")["output"] == engine.model.greedy([9, 8, 3, 4, 5], 1)


@pytest.mark.parametrize("prefix_caching", [False, True])
def test_pressure_preempts_and_recomputes_without_changing_outputs(prefix_caching):
    engine = make(block_size=2, num_blocks=5, max_batch_tokens=6, prefill_chunk_size=2, prefix_caching=prefix_caching)
    prompts = [prompt("aa"), prompt("bb"), prompt("cc")]
    for i, p in enumerate(prompts):
        engine.add(str(i), p, 7)
    reports = drain(engine)
    assert any(e["type"] == "preempted" for e in engine.trace)
    assert any(w["phase"] == "recompute" for r in reports for w in r.work)
    for i, p in enumerate(prompts):
        assert engine.result(str(i))["output"] == engine.model.greedy(p, 7)
    assert engine.stats()["preemptions"] > 0 and engine.stats()["recomputed_tokens"] > 0
    engine.cache.clear_prefixes()
    assert engine.cache.free_pages() == [5]


def test_when_pages_run_out_the_youngest_steps_back_and_the_oldest_never_does():
    engine = make(block_size=2, num_blocks=4, max_batch_tokens=8, prefill_chunk_size=4, prefix_caching=False)
    engine.add("old", prompt("abcd"), 4)
    engine.add("young", prompt("efgh"), 4)
    drain(engine)
    preempted = [e["id"] for e in engine.trace if e["type"] == "preempted"]
    assert preempted and set(preempted) == {"young"}
    assert engine.result("old")["preemptions"] == 0
    # a request preempted while the step was planned brought no tokens to that step
    for e in engine.trace:
        if e["type"] == "preempted":
            tick_tokens = [t for t in engine.trace if t["tick"] == e["tick"] and t["id"] == e["id"] and t["type"] == "token"]
            assert not tick_tokens
    assert engine.result("young")["output"] == engine.model.greedy(prompt("efgh"), 4)


def test_cancel_running_and_queued_requests_without_hurting_a_sibling():
    engine = make(block_size=2, max_sequences=2)
    p = prompt("abc")
    engine.add("A", p, 5)
    engine.step()
    engine.add("B", p, 5)
    engine.step()
    engine.add("queued", p, 1)
    assert engine.cancel("A") and engine.cancel("queued") and not engine.cancel("A")
    drain(engine)
    assert engine.result("A")["status"] == "cancelled" and engine.result("queued")["status"] == "cancelled"
    assert engine.result("B")["output"] == engine.model.greedy(p, 5)
    assert engine.forget("A") and not engine.forget("A")
    engine.cache.clear_prefixes()
    assert engine.cache.free_pages() == [engine.options.num_blocks]


def test_eos_is_emitted_once_counted_and_frees_pages_before_the_limit():
    probe = make()
    first = probe.model.greedy([1, 2], 1)[0]
    engine = make(block_size=2, num_blocks=4, eos=(first,))
    events = list(engine.stream([1, 2], max_new_tokens=5))
    assert [e["token"] for e in events if e["type"] == "token"] == [first]
    assert events[-1] == {"id": events[0]["id"], "type": "finished", "finish_reason": "eos",
                          "usage": {"prompt_tokens": 2, "completion_tokens": 1}}
    assert all(page["active_refs"] == 0 for page in engine.cache.snapshot()["pages"])
    # ignore_eos runs to the length limit
    engine.add("x", [1, 2], 3, ignore_eos=True)
    drain(engine)
    assert engine.result("x")["finish_reason"] == "length" and len(engine.result("x")["output"]) == 3


def test_invalid_inputs_and_requests_that_cannot_fit():
    with pytest.raises(Exception, match="positive integer"):
        make(max_batch_tokens=0)
    engine = make(block_size=2, num_blocks=1, max_sequences=1)
    for bad, pattern in (([], "brings no prompt"), ([-1], r"prompt\[0\] = -1 is no token id"), ([3, 50], r"prompt\[1\] = 50 is no token id")):
        with pytest.raises(ValueError, match=pattern):
            engine.add("x", bad, 1)
    with pytest.raises(ValueError, match="positive integer"):
        engine.add("x", [1], 0)
    with pytest.raises(ValueError, match="more than the whole pool holds"):
        engine.add("x", [1, 2], 2)
    with pytest.raises(ValueError, match="the model has 64"):
        make(num_blocks=64).add("x", [1], 65)
    engine.add("x", [1, 2], 1)
    with pytest.raises(ValueError, match="id of its own"):
        engine.add("x", [1], 1)
    drain(engine)


def test_a_failing_step_ends_every_request_and_returns_every_page():
    engine = make(block_size=2, num_blocks=8)
    engine.add("A", prompt("abcd"), 4)
    engine.add("B", prompt("abcd"), 4)
    engine.step()

    def broken(entries):
        raise RuntimeError("device lost")
    engine.model.step = broken
    with pytest.raises(RuntimeError, match="device lost"):
        engine.step()
    assert not engine.pending
    assert engine.result("A")["status"] == engine.result("B")["status"] == "cancelled"
    assert engine.cache.free_pages() == [8]


def test_generate_returns_outputs_in_order():
    engine = make(max_sequences=2)
    prompts = [prompt("one"), prompt("second"), prompt("3")]
    assert engine.generate(prompts, max_new_tokens=3) == [engine.model.greedy(p, 3) for p in prompts]


# ---- the next decode step launched before the running one is read back ---------------------------------

def make_lookahead(lookahead=True, **kw):
    runner = FakeRunner(kw.pop("block_size", 4), kw.pop("num_blocks", 64), kw.pop("max_sequences", 4), True, kw.pop("eos", ()))
    kw.setdefault("max_batch_tokens", 8)
    kw.setdefault("prefill_chunk_size", 4)
    return Engine(runner, record_trace=True, decode_lookahead=lookahead, **kw)


def test_lookahead_changes_no_output_and_feeds_tokens_on_the_device():
    prompts = {"a": prompt("alpha"), "b": prompt("be"), "c": prompt("gamma ray")}
    limits = {"a": 9, "b": 3, "c": 14}
    probe = make_lookahead(False)
    stop = probe.model.greedy(prompts["a"], 5)[4]          # request a ends early at an end token
    outputs = {}
    for lookahead in (False, True):
        engine = make_lookahead(lookahead)
        for id, p in prompts.items():
            engine.add(id, p, limits[id], stop_token_ids=[stop] if id == "a" else None)
        reports = drain(engine)
        outputs[lookahead] = {id: engine.result(id) for id in prompts}
        assert (engine.model.fed > 0) == lookahead
        assert engine._ahead is None or not any(w.request.status == "running" for w in engine._ahead[0])
        engine.cache.clear_prefixes()
        assert engine.cache.free_pages() == [engine.options.num_blocks]
        ticks = [r.tick for r in reports]
        assert ticks == sorted(set(ticks))
    for id in prompts:
        assert outputs[True][id]["output"] == outputs[False][id]["output"]
        assert outputs[True][id]["finish_reason"] == outputs[False][id]["finish_reason"]
    assert outputs[True]["a"]["finish_reason"] == "eos" and outputs[True]["b"]["finish_reason"] == "length"
    assert outputs[True]["c"]["output"] == probe.model.greedy(prompts["c"], limits["c"])
    want = probe.model.greedy(prompts["a"], limits["a"])
    assert outputs[True]["a"]["output"] == want[:want.index(stop) + 1]


def test_lookahead_with_cancellation_and_a_late_request():
    engine = make_lookahead(True, block_size=2)
    pa, pb, pc = prompt("abc"), prompt("defg"), prompt("hi")
    engine.add("A", pa, 12)
    engine.add("B", pb, 12)
    while not (engine.result("A")["output"] and engine.result("B")["output"]):
        engine.step()
    engine.step()
    assert engine._ahead is not None                      # a step is in flight beyond the one just booked
    assert engine.cancel("A")                             # ... with a share for A, which is thrown away
    engine.add("C", pc, 4)                                # joins after the step in flight
    drain(engine)
    assert engine.result("A")["status"] == "cancelled"
    assert engine.result("B")["output"] == engine.model.greedy(pb, 12)
    assert engine.result("C")["output"] == engine.model.greedy(pc, 4)
    engine.cache.clear_prefixes()
    assert engine.cache.free_pages() == [engine.options.num_blocks]


def test_plan_ahead_only_where_the_next_step_is_certain():
    # somebody waits for admission: the next step is not certain, every step is read back first
    engine = make_lookahead(True, max_sequences=1)
    engine.add("A", prompt("abc"), 6)
    engine.add("B", prompt("de"), 3)
    while engine.result("A")["status"] != "finished":
        engine.step()
        assert engine._ahead is None
    drain(engine)
    assert engine.model.fed > 0                           # B, alone at the end, did run ahead
    # a prompt portion in the batch: not a step of decoded tokens only
    engine = make_lookahead(True)
    engine.add("A", prompt("ab"), 8)
    engine.step(); engine.step()
    engine.add("late", prompt("a long prompt that takes several portions"), 2)
    engine.step()                                         # books the step in flight
    while not engine.result("late")["output"]:
        engine.step()
        assert engine._ahead is None
    drain(engine)
    assert engine.result("A")["output"] == engine.model.greedy(prompt("ab"), 8)
    # no free page for the token after next: nothing is preempted on a guess, the ordinary plan decides
    engine = make_lookahead(True, block_size=2, num_blocks=5, max_sequences=2)
    pa, pb = prompt("abc"), prompt("de")
    engine.add("A", pa, 8)
    engine.add("B", pb, 8)
    reports = drain(engine)
    assert engine.result("A")["output"] == engine.model.greedy(pa, 8)
    assert engine.result("B")["output"] == engine.model.greedy(pb, 8)
    assert engine.stats()["preemptions"] > 0
    assert all(e["type"] != "preempted" or e["id"] == "B" for r in reports for e in r.events)
    # the scheduler itself refuses a step that has not been launched (its tokens are not in the cache yet)
    engine = make_lookahead(False)
    engine.add("A", prompt("ab"), 8)
    engine.step(); engine.step()
    work = engine.scheduler.plan()
    assert [w.phase for w in work] == ["decode"] and engine.scheduler.plan_ahead(work) is None


@pytest.mark.parametrize("seed", range(6))
def test_lookahead_under_random_arrivals_cancellations_and_pressure(seed):
    """Requests arrive, stop at end tokens, are cancelled and preempted at random while steps run ahead: every
    request that finishes has the tokens it would have had alone, and no page is lost."""
    import random
    rng = random.Random(seed)
    num_blocks = rng.choice([6, 9, 16, 40])
    engine = make_lookahead(True, block_size=rng.choice([2, 4]), num_blocks=num_blocks, max_sequences=rng.choice([2, 3, 4]),
                            max_batch_tokens=rng.choice([6, 8, 16]), prefill_chunk_size=rng.choice([2, 4, 8]))
    capacity = num_blocks * engine.options.block_size
    plans, live, cancelled = {}, [], set()
    next_id = steps = 0
    while steps < 400 and (engine.pending or next_id < 12):
        steps += 1
        if next_id < 12 and rng.random() < 0.35:
            p = [rng.randrange(50) for _ in range(rng.randrange(1, 9))]
            limit = rng.randrange(1, 10)
            if len(p) + limit - 1 <= min(capacity, engine.model.max_positions):
                greedy = engine.model.greedy(p, limit)
                stop = greedy[rng.randrange(limit)] if rng.random() < 0.4 else None
                id = f"q{next_id}"
                engine.add(id, p, limit, stop_token_ids=None if stop is None else [stop], ignore_eos=stop is None)
                plans[id] = greedy[:greedy.index(stop) + 1] if stop is not None else greedy
                live.append(id)
            next_id += 1
        if live and rng.random() < 0.05:
            victim = rng.choice(live)
            if engine.cancel(victim):
                cancelled.add(victim)
        report = engine.step()
        assert all(p["refs"] >= 0 and p["active_refs"] >= 0 for p in report.memory["pages"])
        live = [i for i in live if engine.result(i)["status"] in ("waiting", "running")]
    assert not engine.pending
    for id, want in plans.items():
        result = engine.result(id)
        if id in cancelled:
            assert result["status"] == "cancelled" and result["output"] == want[:len(result["output"])]
        else:
            assert result["status"] == "finished" and result["output"] == want, id
    engine.cache.clear_prefixes()
    assert engine.cache.free_pages() == [num_blocks]


def test_mean_walk_of_a_steps_tiles():
    """The hint that the attention kernels get of how unequal the walks of a step's tiles are."""
    from sprout_lm_amd.ops import mean_tile_walk
    assert mean_tile_walk([2048], [2048]) == 1040            # a prompt's first portion: 32, 64, ..., 2,048 keys
    assert mean_tile_walk([2048], [4096]) == 2048 + 1040     # the same after 2,048 earlier tokens
    assert mean_tile_walk([1, 1, 1], [5, 600, 7]) == 0       # decoded tokens have no tiles
    assert mean_tile_walk([1, 40], [900, 40]) == (32 + 64) // 2   # the last tile counts as a whole one
    assert mean_tile_walk([], []) == 0
