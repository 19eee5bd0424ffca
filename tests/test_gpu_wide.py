"""The engine against the plain implementation at the layer widths of the larger models whose throughput is
measured: Qwen2.5-7B sizes (hidden 3,584, 28 heads in 4 groups of head size 128, inner 18,944) and Qwen2.5-32B
sizes (5,120, 40 in 8, 27,648), both with a separate output matrix of 152,064 rows.  At these widths a step takes
other kernels than at the sizes of the other tests: the norm is a kernel of its own, the feed-forward of a decode
step runs on the tiled kernels with K split, the attention groups hold 7 and 5 query heads, the merge of the key
chunks and the output projection are two kernels.  Few layers keep the plain side affordable; every width is whole."""
import numpy as np
import pytest
import torch

from tests import helpers as H
from tests import traces
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

WIDE = {"7b": ("qwen2.5-7b", 2), "32b": ("qwen2.5-32b", 1)}


class Plain:
    """The plain implementation over a folder, with the weights widened to float64 once (its products do that
    on every call otherwise, which at these sizes takes longer than the products)."""

    def __init__(self, folder):
        self.cfg, weights = P.load_folder(folder, "bfloat16")
        self.w = {k: v.astype(np.float64) for k, v in weights.items()}
        self._rows = {}

    def logits(self, dtype, tokens, rows):
        store = P.bf16_round if dtype == "bfloat16" else P.f32
        key = (dtype, tuple(tokens), tuple(rows))
        if key not in self._rows:
            self._rows[key] = P.forward_logits(self.w, self.cfg, list(tokens), store=store, rows=list(rows))
        return self._rows[key]


def bound(dtype, want):
    if dtype == "float32":     # the reference's bound for real checkpoints (test/model.integration.ts:69)
        return 1e-3 + 1e-4 * np.abs(want)
    return H.tolerance(dtype, want)


@pytest.fixture(scope="module", params=sorted(WIDE))
def wide(request, tmp_path_factory):
    import sprout_lm_amd as S
    from sprout_lm_amd.cli import PRESETS
    from sprout_lm_amd.weights import write_model_folder
    preset, layers = WIDE[request.param]
    raw = dict(PRESETS[preset], num_hidden_layers=layers, max_position_embeddings=2048)
    folder = str(tmp_path_factory.mktemp(f"wide_{request.param}"))
    write_model_folder(folder, S.config_from_dict(raw), seed=31, dtype=torch.bfloat16, std=0.02)
    return folder, raw, Plain(folder)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_mixed_replay_and_recorded_decode_at_the_widths_of_the_larger_models(wide, dtype):
    """A mixed replay (up to four live requests, portions beside single tokens, a pool so small that pages are used
    again), then decode steps through recorded graphs with a batch that is no power of two and contexts that cross
    256 keys: every row of logits against the plain implementation."""
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.engine.trace import TraceSession
    from sprout_lm_amd.sampling import SamplingParams
    folder, raw, plain = wide
    vocab = raw["vocab_size"]
    requests = {f"r{i}": H.random_tokens(vocab, n, 700 + i) for i, n in enumerate([70, 40, 130, 33, 90])}
    trace = traces.mixed(requests, seed=13)
    pool_tokens = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    runner = ModelRunner.from_folder(folder, dtype, block_size=16, num_blocks=pool_tokens // 16, max_sequences=4)
    session = TraceSession(runner)
    owners, worst = {}, 0.0
    for record, rows in zip(trace.steps, trace.expected):
        logits = session.run_step(record)
        for rid, seq in session.live.items():
            for page in seq.blocks[0]:
                if rid not in owners.setdefault(page, []):
                    owners[page].append(rid)
        if not rows:
            continue
        got = logits.cpu().numpy()
        by_request = {}
        for i, (rid, pos) in enumerate(rows):
            by_request.setdefault(rid, []).append((i, pos))
        for rid, places in by_request.items():
            want = plain.logits(dtype, requests[rid][:max(p for _, p in places) + 1], [p for _, p in places])
            for (i, pos), ref in zip(places, want):
                err = np.abs(got[i] - ref)
                worst = max(worst, float((err / bound(dtype, ref)).max()))
                assert np.all(err <= bound(dtype, ref)), f"replay {rid} position {pos}: {err.max():.3e}"
    assert sum(len(r) > 1 for r in owners.values()) >= 2, "no page of the pool served two requests"
    assert runner.cache.free_pages() == [pool_tokens // 16] and not session.live
    del session, runner
    torch.cuda.empty_cache()

    # recorded decode: three requests (a step of four rows, one of them padding), contexts 250.. and 253.. cross 256
    prompts = {"a": H.random_tokens(vocab, 250, 801), "b": H.random_tokens(vocab, 40, 802), "c": H.random_tokens(vocab, 253, 803)}
    runner = ModelRunner.from_folder(folder, dtype, block_size=16, num_blocks=64, max_sequences=3)
    seqs = {k: runner.cache.create() for k in prompts}
    history = {k: list(v) for k, v in prompts.items()}
    for k, tokens in prompts.items():               # whole prompts but their last token, eagerly, no logits
        assert runner.cache.reserve(seqs[k], len(tokens) - 1)
        runner.step([StepEntry(seqs[k], tokens[:-1], [])])
    steps, rows = 12, {k: [] for k in prompts}
    for _ in range(steps):
        entries = []
        for k in prompts:
            assert runner.cache.reserve(seqs[k], seqs[k].length + 1)
            entries.append(StepEntry(seqs[k], [history[k][seqs[k].length]], [0]))
        pending = runner.launch_decode(entries, [SamplingParams()] * 3, [0] * 3)
        assert pending is not None, "the step did not run from a recorded graph"
        tokens = runner.finish_decode(pending)
        got = pending.logits[:3].cpu().numpy()
        for k, token, row in zip(prompts, tokens, got):
            assert token == int(np.argmax(row))
            rows[k].append(row)
            history[k].append(token)                # greedy: the next step feeds what this one chose
    assert runner._graphs.replays == steps
    for k in prompts:
        first = len(prompts[k]) - 1
        want = plain.logits(dtype, history[k][:-1], list(range(first, first + steps)))
        for i, (row, ref) in enumerate(zip(rows[k], want)):
            err = np.abs(row - ref)
            worst = max(worst, float((err / bound(dtype, ref)).max()))
            assert np.all(err <= bound(dtype, ref)), f"recorded decode {k} position {first + i}: {err.max():.3e}"
    del runner
    torch.cuda.empty_cache()

    if dtype == "bfloat16" and raw["hidden_size"] == 3584:
        # one prompt of 2,048 tokens in one step, the size whose throughput is measured: the products' largest block
        # shapes (q/k/v on blocks of 256 x 160 followed by the rotation kernel, the gated product on 256 x 256) and
        # the prompt attention's long walks, tiles taken in pairs
        tokens = H.random_tokens(vocab, 2048, 900)
        places = [0, 255, 256, 1500, 2047]
        runner = ModelRunner.from_folder(folder, dtype, block_size=16, num_blocks=130, max_sequences=1)
        seq = runner.cache.create()
        assert runner.cache.reserve(seq, len(tokens))
        got = runner.step([StepEntry(seq, tokens, places)]).cpu().numpy()
        want = plain.logits(dtype, tokens, places)
        for row, ref, pos in zip(got, want, places):
            err = np.abs(row - ref)
            worst = max(worst, float((err / bound(dtype, ref)).max()))
            assert np.all(err <= bound(dtype, ref)), f"long prompt position {pos}: {err.max():.3e}"
        seq.release()
    print(f"wide {raw['hidden_size']} {dtype}: worst {worst:.2f} of the bound")
