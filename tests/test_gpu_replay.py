"""Replay of the same requests cut into steps in different ways, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import helpers as H
from tests import traces

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("models"))
    return {name: H.make_model_folder(root, name) for name in H.CONFIGS}


def requests_for(name, lengths, seed=100):
    vocab = H.CONFIGS[name]["vocab_size"]
    return {f"r{i}": H.random_tokens(vocab, n, seed + i) for i, n in enumerate(lengths)}


def replay_in_process(folder, name, dtype, trace, max_tokens, page=None, num_blocks=None, reused=None):
    """Drive the engine's TraceSession directly; returns per step the logits rows (or None).
    `reused`: a dict that receives, per physical page that served more than one request, those requests."""
    from sprout_lm_amd.engine import ModelRunner
    from sprout_lm_amd.engine.trace import TraceSession
    page = page or H.PAGE_SIZE[name]
    runner = ModelRunner.from_folder(folder, dtype, block_size=page, num_blocks=num_blocks or -(-max_tokens // page),
                                     max_sequences=8)
    session = TraceSession(runner)
    out = []
    owners: dict = {}                      # physical page -> requests that held it, in order
    for record in trace.steps:
        logits = session.run_step(record)
        out.append(None if logits is None or not logits.shape[0] else logits.cpu().numpy().copy())
        holders = {}
        for rid, seq in session.live.items():
            for page_id in seq.blocks[0]:
                assert holders.setdefault(page_id, rid) == rid, f"page {page_id} is held by two requests at once"
                if rid not in owners.setdefault(page_id, []):
                    owners[page_id].append(rid)
    if reused is not None:
        reused.update({p: r for p, r in owners.items() if len(r) > 1})
        assert len(owners) <= runner.cache.num_blocks
    assert runner.cache.free_pages() == [runner.cache.num_blocks], "pages were lost"
    assert not session.live
    return out


def check(folder, dtype, requests, trace, results):
    worst = 0.0
    for step, (rows, got) in enumerate(zip(trace.expected, results)):
        if not rows:
            assert got is None
            continue
        assert got.shape[0] == len(rows)
        for i, (rid, pos) in enumerate(rows):
            want = H.plain_logits(folder, dtype, requests[rid])[pos]
            err = float(np.abs(got[i] - want).max())
            worst = max(worst, err)
            assert err <= H.tolerance(dtype, want), f"step {step} request {rid} position {pos}: error {err:.3e}"
    return worst


LENGTHS = {"A": [5, 17, 33, 70, 128, 64], "B": [1, 9, 40, 70, 97, 33, 2], "C": [48, 130, 65, 200, 90, 33]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "portions", "mixed"])
def test_replay_family(folders, name, dtype, family):
    requests = requests_for(name, LENGTHS[name])
    roomy = 4 * 64 * (1 + max(LENGTHS[name]) // 64)
    if family == "whole":
        trace, pool = traces.whole(requests), roomy
    elif family == "tail":
        trace, pool = traces.tail_decoded(requests), roomy
    elif family == "portions":
        trace, pool = traces.portions(requests), roomy
    else:
        # the pool holds exactly four requests rounded up to 64 tokens: pages are used again
        trace = traces.mixed(requests, seed=7)
        pool = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    reused = {}
    results = replay_in_process(folders[name], name, dtype, trace, pool, reused=reused)
    if family == "mixed":     # what the family is for: later requests compute in pages that earlier ones gave back
        assert len(reused) >= 2, "no page of the pool served two requests"
    worst = check(folders[name], dtype, requests, trace, results)
    print(f"{family} {name} {dtype}: {len(trace.steps)} steps, worst error {worst:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page", [("A", 12), ("B", 20), ("C", 6)])
def test_replay_with_pages_of_odd_sizes(folders, name, dtype, page):
    """Pages whose size is no power of two (and, at 6, no multiple of 4): other attention kernels take over.
    The pool holds the four longest requests and no page more, so pages are used again."""
    requests = requests_for(name, LENGTHS[name], seed=300)
    trace = traces.mixed(requests, seed=11)
    pages = sum(sorted(-(-len(t) // page) for t in requests.values())[-4:])
    reused = {}
    results = replay_in_process(folders[name], name, dtype, trace, None, page=page, num_blocks=pages, reused=reused)
    assert len(reused) >= 2, "no page of the pool served two requests"
    check(folders[name], dtype, requests, trace, results)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_agree_with_each_other(folders, dtype):
    """Whole, token-by-token and portioned replays give the same logits beyond rounding."""
    name = "B"
    requests = requests_for(name, [70])
    by_family = {}
    for family, trace in (("whole", traces.whole(requests)), ("tail", traces.tail_decoded(requests, tail=69)),
                          ("portions", traces.portions(requests))):
        results = replay_in_process(folders[name], name, dtype, trace, 256)
        rows = {}
        for expect, got in zip(trace.expected, results):
            for i, key in enumerate(expect):
                rows[key] = got[i]
        by_family[family] = rows
    bound = 1e-5 if dtype == "float32" else 3e-2
    for key, row in by_family["whole"].items():
        for other in ("tail", "portions"):
            if key in by_family[other]:
                assert np.abs(row - by_family[other][key]).max() <= bound * max(1.0, np.abs(row).max())


def test_trace_run_program(folders, tmp_path):
    """bin/trace_run as a user runs it: stdin lines in, `done` lines and .f32 files out."""
    name, dtype = "A", "float32"
    requests = requests_for(name, [33, 70, 20, 64, 45])
    trace = traces.mixed(requests, seed=3)
    pool = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    out = tmp_path / "logits"
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name],
                             "--dtype", dtype, "--out", str(out), "--max-tokens", str(pool)],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for record in trace.steps:
            proc.stdin.write(json.dumps(record) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {record['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    vocab = H.CONFIGS[name]["vocab_size"]
    results = []
    for record, rows in zip(trace.steps, trace.expected):
        path = out / f"{record['step']}.f32"
        if rows:
            results.append(np.fromfile(path, dtype="<f4").reshape(len(rows), vocab))
        else:
            assert not path.exists()
            results.append(None)
    check(folders[name], dtype, requests, trace, results)
    # the index names the request and position of every row, as the trace's builder knows them
    index = [json.loads(line) for line in open(out / "index.jsonl")]
    assert [r["step"] for r in index] == [s["step"] for s, rows in zip(trace.steps, trace.expected) if rows]
    for record in index:
        assert [(r["request"], r["position"]) for r in record["rows"]] == trace.expected[record["step"]]
        assert [r["row"] for r in record["rows"]] == list(range(len(record["rows"])))
    # the plain side of the same trace, file by file
    from tests.plain import trace_plain
    cfg, weights = H.plain_model(folders[name], dtype)
    trace_plain.replay(cfg, weights, dtype, trace.steps[:12], str(tmp_path / "plain"))
    plain_index = [json.loads(line) for line in open(tmp_path / "plain" / "index.jsonl")]
    assert plain_index == index[:len(plain_index)] and plain_index
    for record in plain_index:
        want = np.fromfile(tmp_path / "plain" / record["file"], dtype="<f4")
        got = np.fromfile(out / record["file"], dtype="<f4")
        assert want.shape == got.shape and np.abs(want - got).max() <= H.tolerance(dtype, want)
