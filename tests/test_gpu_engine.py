"""Generation through the engine's entry points on the GPU, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import helpers as H
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("models"))
    return {name: H.make_model_folder(root, name) for name in ("A", "B")}


def plain_greedy(folder, dtype, prompt, steps):
    """Greedy continuation by the plain implementation; also returns the smallest top-2 margin."""
    history, out, margin = list(prompt), [], np.inf
    for _ in range(steps):
        row = H.plain_logits(folder, dtype, history)[-1]
        top = np.sort(row)[-2:]
        margin = min(margin, float(top[1] - top[0]))
        token = int(np.argmax(row))
        history.append(token)
        out.append(token)
    return out, margin


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    """Tiny A: 3 requests with prompts 5/17/33 and 8 greedy steps; tiny B: prompts 1/9/40/70 in portions of 16.

    Every generated token is held to the plain implementation's logits for the same history: it is their
    largest, or, where reduced precision may take the other side of a near tie, within the logits' error bound
    of the largest.  Most tokens must be the largest outright."""
    from sprout_lm_amd.engine import Engine
    tokens = best = 0
    for name, lengths, steps, chunk in (("A", (5, 17, 33), 8, 64), ("B", (1, 9, 40, 70), 12, 16)):
        engine = Engine.from_folder(folders[name], dtype, block_size=H.PAGE_SIZE[name], num_blocks=64, max_sequences=4,
                                    max_batch_tokens=48, prefill_chunk_size=chunk, record_trace=True)
        vocab = H.CONFIGS[name]["vocab_size"]
        prompts = [H.random_tokens(vocab, n, 40 + i) for i, n in enumerate(lengths)]
        outputs = engine.generate(prompts, max_new_tokens=steps, ignore_eos=True)
        for prompt, got in zip(prompts, outputs):
            assert len(got) == steps
            history = list(prompt)
            for i, token in enumerate(got):
                row = H.plain_logits(folders[name], dtype, history)[-1]
                top = int(np.argmax(row))
                tokens += 1
                if token == top:
                    best += 1
                else:
                    slack = 2 * H.tolerance(dtype, row)
                    assert row[top] - row[token] <= slack, \
                        f"{name} prompt of {len(prompt)}, token {i}: {token} is {row[top] - row[token]:.3e} below the best"
                history.append(token)
        engine.cache.clear_prefixes()
        assert engine.cache.free_pages() == [64]
    print(f"greedy {dtype}: {best} of {tokens} tokens are the plain side's largest logit")
    assert best == tokens if dtype == "float32" else best >= 0.9 * tokens


def test_scheduling_never_changes_generation(folders):
    """Pressure (preemption and recompute), prefix sharing and a late arrival give the solo outputs (float32)."""
    from sprout_lm_amd.engine import Engine
    name, dtype = "B", "float32"
    vocab = H.CONFIGS[name]["vocab_size"]
    shared = H.random_tokens(vocab, 24, 77)
    prompts = {"A": shared + H.random_tokens(vocab, 9, 78), "B": shared + H.random_tokens(vocab, 5, 79),
               "C": H.random_tokens(vocab, 40, 80), "D": H.random_tokens(vocab, 3, 81)}
    want = {k: plain_greedy(folders[name], dtype, p, 12)[0] for k, p in prompts.items()}
    for num_blocks, expect_preemption in ((64, False), (12, True)):
        engine = Engine.from_folder(folders[name], dtype, block_size=8, num_blocks=num_blocks, max_sequences=4,
                                    max_batch_tokens=24, prefill_chunk_size=16, record_trace=True)
        engine.add("A", prompts["A"], 12, ignore_eos=True)
        engine.step(); engine.step(); engine.step()
        for k in "BCD":
            engine.add(k, prompts[k], 12, ignore_eos=True)
        ticks = 0
        while engine.pending:
            ticks += 1
            assert ticks < 2000
            report = engine.step()
            assert sum(w["tokens"] for w in report.work) <= 24
        for k in prompts:
            assert engine.result(k)["output"] == want[k], f"request {k} with {num_blocks} pages"
        assert engine.result("B")["prefix_hits"] >= 8
        assert any(e["type"] == "preempted" for e in engine.trace) == expect_preemption
        assert all(p["active_refs"] == 0 for p in engine.cache.snapshot()["pages"])
        engine.cache.clear_prefixes()
        assert engine.cache.free_pages() == [num_blocks]


def test_temperature_sampling_is_reproducible_and_independent_of_the_batch(folders):
    from sprout_lm_amd.engine import Engine
    name = "A"
    vocab = H.CONFIGS[name]["vocab_size"]
    prompt = H.random_tokens(vocab, 12, 5)

    def run(extra, seed):
        engine = Engine.from_folder(folders[name], "float32", block_size=16, num_blocks=32, max_sequences=4,
                                    max_batch_tokens=32, prefill_chunk_size=8)
        for i in range(extra):
            engine.add(f"other{i}", H.random_tokens(vocab, 7 + 3 * i, 50 + i), 10, temperature=1.0, seed=99 + i, ignore_eos=True)
        engine.add("me", prompt, 10, temperature=1.5, seed=seed, ignore_eos=True)
        while engine.pending:
            engine.step()
        return engine.result("me")["output"]

    alone = run(0, 1234)
    assert run(0, 1234) == alone and run(3, 1234) == alone
    assert run(0, 4321) != alone
    greedy = plain_greedy(folders[name], "float32", prompt, 10)[0]
    assert alone != greedy            # a temperature of 1.5 over 256 tokens leaves the greedy path


def test_command_line_generate_and_demo(folders, tmp_path):
    report = tmp_path / "report.json"
    env = dict(os.environ, MAX_NEW_TOKENS="5", REPORT_PATH=str(report))
    done = subprocess.run([sys.executable, "-m", "sprout_lm_amd", "generate", folders["A"], "--prompt-ids", "3,1,4,1,5,9,2,6",
                           "--dtype", "float32", "--ignore-eos"], cwd=ROOT, env=env, capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr
    final = json.loads(done.stdout.strip().splitlines()[-1])
    assert final["phase"] == "finished" and len(final["output"]) == 5
    assert final["output"] == plain_greedy(folders["A"], "float32", [3, 1, 4, 1, 5, 9, 2, 6], 5)[0]
    assert json.load(open(report))["output"] == final["output"]
    shown = {}
    for mode in ("--pressure", None):
        demo = subprocess.run([sys.executable, "-m", "sprout_lm_amd", "demo", "--json"] + ([mode] if mode else []), cwd=ROOT,
                              capture_output=True, text=True, timeout=120)
        assert demo.returncode == 0, demo.stderr
        shown[mode] = json.loads(demo.stdout)
        results = shown[mode]["results"]
        assert [results[k]["status"] for k in ("long", "short", "twin", "late")] == ["finished"] * 4
        assert [len(results[k]["output"]) for k in ("long", "short", "twin", "late")] == [10, 12, 8, 6]
    roomy, tight = shown[None], shown["--pressure"]
    assert tight["mode"] == "pressure" and tight["stats"]["preemptions"] > 0 and tight["stats"]["recomputed_tokens"] > 0
    assert roomy["stats"]["preemptions"] == 0 and roomy["results"]["twin"]["prefix_hits"] == 16
    # what the demo is there to show: a round whose one batch mixes a portion of a prompt with decoded tokens,
    # rounds replayed from a recorded graph, and rounds whose successor was launched before they were read back
    assert any({w["phase"] for w in r["work"]} >= {"prefill", "decode"} for r in roomy["rounds"])
    assert roomy["graph_replays"] > 0 and any(r["next_round_already_launched"] for r in roomy["rounds"])
    # scheduling changes nothing of what the greedy requests generate
    for k in ("long", "short", "twin"):
        assert tight["results"][k]["output"] == roomy["results"][k]["output"]
    text = subprocess.run([sys.executable, "-m", "sprout_lm_amd", "demo"], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert text.returncode == 0 and "graph replay, bucket" in text.stdout and "what came out:" in text.stdout


def test_first_tokens_and_long_decoding(folders):
    """The first tokens of a sequence (positions 0, 1, 2 fed one by one) and 200 decoded tokens in a row."""
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    name = "B"
    vocab = H.CONFIGS[name]["vocab_size"]
    tokens = H.random_tokens(vocab, 230, 9)
    for dtype in ("float32", "bfloat16"):
        runner = ModelRunner.from_folder(folders[name], dtype, block_size=8, num_blocks=40, max_sequences=2)
        seq = runner.cache.create()
        want = H.plain_logits(folders[name], dtype, tokens)
        worst = 0.0
        for p, token in enumerate(tokens):
            assert runner.cache.reserve(seq, p + 1)
            got = runner.step([StepEntry(seq, [token], [0])]).cpu().numpy()[0]
            worst = max(worst, float(np.abs(got - want[p]).max()))
            assert np.abs(got - want[p]).max() <= H.tolerance(dtype, want[p]), f"{dtype} position {p}"
        print(f"long decode {dtype}: worst {worst:.3e}")
        seq.release()


def test_graph_replays_equal_eager_steps(folders):
    """Decode steps replayed from a recorded graph give the tokens of eagerly launched steps, replay after
    replay, with eager prompt steps and synchronisations in between (requests arrive while others decode)."""
    from sprout_lm_amd.engine import Engine
    name = "A"
    vocab = H.CONFIGS[name]["vocab_size"]
    prompts = [H.random_tokens(vocab, n, 60 + i) for i, n in enumerate((7, 21, 3, 40, 12))]

    def run(use_graphs):
        engine = Engine.from_folder(folders[name], "bfloat16", block_size=16, num_blocks=48, max_sequences=4,
                                    max_batch_tokens=32, prefill_chunk_size=16)
        engine.model.use_graphs = use_graphs
        engine.add("r0", prompts[0], 30, ignore_eos=True)
        engine.add("r1", prompts[1], 25, ignore_eos=True)
        steps = 0
        while engine.pending:
            steps += 1
            if steps == 6:
                engine.add("r2", prompts[2], 20, temperature=0.8, seed=5, ignore_eos=True)
            if steps == 15:
                engine.add("r3", prompts[3], 10, ignore_eos=True)
                engine.add("r4", prompts[4], 28, temperature=1.2, seed=9, ignore_eos=True)
            engine.step()
        replays = engine.model._graphs.replays if engine.model._graphs else 0
        return [engine.result(f"r{i}")["output"] for i in range(5)], replays

    eager, none = run(False)
    graphed, replays = run(True)
    assert none == 0 and replays > 40
    assert graphed == eager


def test_lookahead_equals_synchronous_steps(folders):
    """The next decode step launched before the running one is read back (tokens go from step to step on the
    device) gives every request the tokens of steps that each wait for their result: greedy and with
    temperature, requests of different lengths, one arriving under way."""
    from sprout_lm_amd.engine import Engine
    name = "A"
    vocab = H.CONFIGS[name]["vocab_size"]
    prompts = [H.random_tokens(vocab, n, 40 + i) for i, n in enumerate((6, 19, 33, 4))]

    def run(lookahead, max_graphs=None):
        engine = Engine.from_folder(folders[name], "bfloat16", block_size=16, num_blocks=48, max_sequences=4,
                                    max_batch_tokens=32, prefill_chunk_size=16, decode_lookahead=lookahead)
        if max_graphs is not None:        # so few that recorded graphs are dropped and recorded again under way
            from sprout_lm_amd.engine.graphs import DecodeGraphs
            engine.model._graphs = DecodeGraphs(engine.model, max_graphs=max_graphs)
        engine.add("r0", prompts[0], 40, ignore_eos=True)
        engine.add("r1", prompts[1], 22, temperature=0.7, seed=11, ignore_eos=True)
        engine.add("r2", prompts[2], 9, ignore_eos=True)
        steps = ahead = 0
        while engine.pending:
            steps += 1
            if steps == 25:
                engine.add("r3", prompts[3], 14, ignore_eos=True)
            engine.step()
            ahead += engine._ahead is not None
        return [engine.result(f"r{i}")["output"] for i in range(4)], ahead

    sync, none = run(False)
    overlapped, launched = run(True)
    assert none == 0 and launched > 20
    assert overlapped == sync
    crowded, launched = run(True, max_graphs=1)
    assert launched > 20 and crowded == sync


def test_lookahead_steps_give_the_tokens_of_synchronous_steps(folders):
    """With the next decode step launched before the running one is read back (tokens go from step to step on
    the device) every request gets the tokens it gets when each step waits for its result: greedy and with
    temperature, with an end token that stops one request early, arrivals, a cancellation, and context buckets
    that change under way."""
    from sprout_lm_amd.engine import Engine
    name = "C"
    vocab = H.CONFIGS[name]["vocab_size"]
    folder = H.make_model_folder(os.path.dirname(folders["A"]), name)
    prompts = [H.random_tokens(vocab, n, 90 + i) for i, n in enumerate((5, 30, 250, 9, 17))]

    def run(lookahead, stop=None):
        engine = Engine.from_folder(folder, "bfloat16", block_size=16, num_blocks=64, max_sequences=4,
                                    max_batch_tokens=64, prefill_chunk_size=32, decode_lookahead=lookahead)
        engine.add("r0", prompts[0], 60, ignore_eos=True)
        engine.add("r1", prompts[1], 40, stop_token_ids=None if stop is None else [stop])
        engine.add("r2", prompts[2], 25, temperature=0.9, seed=3, ignore_eos=True)     # crosses 256 keys
        steps, ahead = 0, 0
        while engine.pending:
            steps += 1
            if steps == 20:
                engine.add("r3", prompts[3], 30, ignore_eos=True)
            if steps == 30:
                engine.cancel("r0")
                engine.add("r4", prompts[4], 12, temperature=0.5, seed=1, ignore_eos=True)
            engine.step()
            ahead += engine._ahead is not None
        engine.cache.clear_prefixes()
        assert engine.cache.free_pages() == [64] * len(engine.cache.free_pages())
        return {f"r{i}": engine.result(f"r{i}") for i in range(5)}, ahead

    first, _ = run(False)
    stop = first["r1"]["output"][11]
    sync, none = run(False, stop)
    ahead, launched = run(True, stop)
    assert none == 0 and launched > 30
    assert sync["r1"]["finish_reason"] == "eos" and len(sync["r1"]["output"]) <= 12
    for k in ("r1", "r2", "r3", "r4"):
        assert ahead[k]["output"] == sync[k]["output"] and ahead[k]["finish_reason"] == sync[k]["finish_reason"], k
    assert ahead["r0"]["status"] == "cancelled"
    n = min(len(ahead["r0"]["output"]), len(sync["r0"]["output"]))
    assert n > 5 and ahead["r0"]["output"][:n] == sync["r0"]["output"][:n]


def test_real_layer_sizes_both_dtypes(tmp_path):
    """Two layers with the sizes of Qwen2.5-0.5B (hidden 896, 14 heads in 2 groups of head size 64, inner 4864,
    vocabulary 151936, tied): whole prompt, portions and single tokens against the plain implementation."""
    import torch
    import sprout_lm_amd as S
    from sprout_lm_amd.cli import PRESETS
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.weights import write_model_folder
    raw = dict(PRESETS["qwen2.5-0.5b"], num_hidden_layers=2)
    folder = str(tmp_path / "half_b")
    write_model_folder(folder, S.config_from_dict(raw), seed=8, dtype=torch.bfloat16, std=0.02)
    tokens = H.random_tokens(raw["vocab_size"], 83, 17)
    for dtype in ("float32", "bfloat16"):
        want = H.plain_logits(folder, dtype, tokens)
        runner = ModelRunner.from_folder(folder, dtype, block_size=16, num_blocks=16, max_sequences=2)
        seq = runner.cache.create()
        rows = {}
        fed = 0
        for n in (40, 17, 2, 1, 1, 16, 1, 1, 1, 1, 1, 1):
            assert runner.cache.reserve(seq, fed + n)
            got = runner.step([StepEntry(seq, tokens[fed:fed + n], [0, n - 1] if n > 1 else [0])]).cpu().numpy()
            rows[fed] = got[0]
            rows[fed + n - 1] = got[-1]
            fed += n
        assert fed == len(tokens)
        for pos, row in rows.items():
            err = np.abs(row - want[pos])
            if dtype == "float32":   # the reference's bound for real checkpoints (test/model.integration.ts:69)
                assert np.all(err <= 1e-3 + 1e-4 * np.abs(want[pos])), f"position {pos}: {err.max():.3e}"
            else:
                assert err.max() <= H.tolerance(dtype, want[pos]), f"position {pos}: {err.max():.3e}"
        seq.release()


@pytest.mark.parametrize("block", range(4))
def test_random_scheduling_never_changes_generation(folders, block):
    """Random page sizes, pools down to one request's need, budgets, portions, arrivals, cancellations,
    prefix sharing, look-ahead on and off and as few as one recorded graph: every request generates what it
    generates alone (float32, where no near tie can fall the other way), and no page is lost."""
    import random
    from sprout_lm_amd.engine import Engine
    from sprout_lm_amd.engine.graphs import DecodeGraphs

    def alone(name, r):
        engine = Engine.from_folder(folders[name], "float32", block_size=16, num_blocks=16, max_sequences=1,
                                    max_batch_tokens=256, prefill_chunk_size=256, prefix_caching=False,
                                    decode_lookahead=False)
        engine.add("s", r["prompt"], r["max_new"], temperature=r["temperature"], seed=r["seed"], stop_token_ids=r["stops"])
        while engine.pending:
            engine.step()
        output = engine.result("s")["output"]
        engine.close()
        return output

    for case in range(8 * block, 8 * block + 8):
        rng = random.Random(4000 + case)
        name = rng.choice("AB")
        vocab = H.CONFIGS[name]["vocab_size"]
        page = rng.choice([4, 8, 12, 16, 32])
        shared = H.random_tokens(vocab, rng.randint(0, 40), case)
        requests = []
        for i in range(rng.randint(2, 6)):
            prompt = (shared[:rng.randint(0, len(shared))] + H.random_tokens(vocab, rng.randint(1, 60), 7 * case + i))[:90]
            requests.append(dict(id=f"r{i}", prompt=prompt, max_new=rng.randint(1, 20), temperature=rng.choice([0.0, 0.0, 0.8]),
                                 seed=rng.randrange(1 << 30), arrive=rng.randint(0, 10),
                                 stops=rng.choice([None, None, [rng.randrange(vocab), rng.randrange(vocab)]]),
                                 cancel=rng.choice([None, None, None, rng.randint(1, 25)])))
        need = max(-(-(len(r["prompt"]) + r["max_new"]) // page) for r in requests)
        num_blocks = rng.randint(need, need * rng.randint(1, 4))
        engine = Engine.from_folder(folders[name], "float32", block_size=page, num_blocks=num_blocks,
                                    max_sequences=rng.randint(1, 6), max_batch_tokens=rng.choice([8, 16, 48, 256]),
                                    prefill_chunk_size=rng.choice([2, 5, 16, 64]), prefix_caching=rng.random() < 0.6,
                                    decode_lookahead=rng.random() < 0.7)
        engine.model._graphs = DecodeGraphs(engine.model, max_graphs=rng.choice([1, 2, 32]))
        tick, cancelled, waiting = 0, set(), sorted(requests, key=lambda r: r["arrive"])
        while waiting or engine.pending:
            while waiting and waiting[0]["arrive"] <= tick:
                r = waiting.pop(0)
                engine.add(r["id"], r["prompt"], r["max_new"], temperature=r["temperature"], seed=r["seed"],
                           stop_token_ids=r["stops"])
            for r in requests:
                known = engine.scheduler.requests.get(r["id"])
                if r["cancel"] == tick and known is not None and known.status in ("waiting", "running"):
                    engine.cancel(r["id"])
                    cancelled.add(r["id"])
            engine.step()
            tick += 1
            assert tick < 2000, f"case {case}: no progress"
        for r in requests:
            got, want = engine.result(r["id"])["output"], alone(name, r)
            assert got == (want[:len(got)] if r["id"] in cancelled else want), f"case {case}, request {r['id']}"
        engine.cache.clear_prefixes()
        assert engine.cache.free_pages() == [num_blocks], f"case {case}: pages were lost"
        engine.close()
