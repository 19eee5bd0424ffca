"""Steps replayed from recorded HIP graphs, compared by their logits with the plain implementation.

Generation runs every step of single tokens through `ModelRunner.launch_decode`; the other logits tests step
eagerly.  Here the recorded path itself is held to the plain side: its own descriptor builder, padded rows,
context buckets, and the kernels that only steps of decoded tokens take at real layer sizes."""
import numpy as np
import pytest
import torch

from tests import helpers as H
from tests.plain import qwen2_plain as P

pytestmark = pytest.mark.gpu


def plain_rows(folder, tokens, rows):
    """bfloat16-rounded plain logits of `tokens` at `rows`, with the weights widened once (exactly) to float64."""
    cfg, w = H.plain_model(folder, "bfloat16")
    key = ("f64", folder)
    if key not in H._PLAIN_CACHE:
        H._PLAIN_CACHE[key] = {k: v.astype(np.float64) for k, v in w.items()}
    return P.forward_logits(H._PLAIN_CACHE[key], cfg, list(tokens), store=P.bf16_round, rows=rows)


def decode_through_graphs(runner, seqs, tokens, fed, steps, folder, label):
    """Feed token `fed[r]` of every request r in `seqs` as one recorded step, `steps` times; compare the step's
    logits with the plain implementation.  Returns the worst error as a fraction of the bound."""
    from sprout_lm_amd.engine import StepEntry
    from sprout_lm_amd.sampling import SamplingParams
    worst = 0.0
    for _ in range(steps):
        names = list(seqs)
        entries = []
        for r in names:
            assert runner.cache.reserve(seqs[r], fed[r] + 1)
            entries.append(StepEntry(seqs[r], [tokens[r][fed[r]]], [0]))
        pending = runner.launch_decode(entries, [SamplingParams()] * len(names), [0] * len(names))
        assert pending is not None, "the step did not run from a recorded graph"
        sampled = runner.finish_decode(pending)
        got = pending.logits[:len(names)].cpu().numpy()
        for i, r in enumerate(names):
            want = plain_rows(folder, tokens[r][:fed[r] + 1], [fed[r]])[0]
            err = float(np.abs(got[i] - want).max()) / H.tolerance("bfloat16", want)
            worst = max(worst, err)
            assert err <= 1.0, f"{label}: request {r} at position {fed[r]}: {err:.2f} of the bound"
            if want.max() - np.partition(want, -2)[-2] > 2 * H.tolerance("bfloat16", want):
                assert sampled[i] == int(np.argmax(want)), f"{label}: request {r} at position {fed[r]}: sampled token"
            fed[r] += 1
    return worst


def test_recorded_steps_of_many_sequences_rotate_by_their_own_positions(tmp_path):
    """More than 64 sequences in a step take the tiled q/k/v product whose epilogue rotates by a table of sines
    and cosines that the first layer of a step computes.  A recorded step must compute that table anew at every
    replay: 530 sequences at different positions, four replays, every logit row against the plain side."""
    import sprout_lm_amd as S
    from sprout_lm_amd import ops
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.weights import write_model_folder
    raw = dict(model_type="qwen2", hidden_act="silu", hidden_size=1280, intermediate_size=256, num_hidden_layers=1,
               num_attention_heads=10, num_key_value_heads=5, vocab_size=300, max_position_embeddings=64,
               rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=True, eos_token_id=0)
    n, steps = 530, 4
    # the case this test is for: at the recorded step's 1,024 rows the projection rotates in its epilogue
    assert ops.fused_supported(ops.FUSED_ROPE, 1024, (10 + 2 * 5) * 128, 1280, 128, 128, False)
    folder = str(tmp_path / "wide")
    write_model_folder(folder, S.config_from_dict(raw), seed=21, dtype=torch.bfloat16, std=0.03)
    rng = np.random.default_rng(5)
    tokens = {r: [int(t) for t in rng.integers(0, 300, int(rng.integers(1, 7)) + steps)] for r in range(n)}
    runner = ModelRunner.from_folder(folder, "bfloat16", block_size=16, num_blocks=n + 8, max_sequences=n)
    seqs = {r: runner.cache.create() for r in range(n)}
    fed = {r: len(tokens[r]) - steps for r in range(n)}
    entries = []
    for r in range(n):
        assert runner.cache.reserve(seqs[r], fed[r])
        entries.append(StepEntry(seqs[r], tokens[r][:fed[r]], []))
    assert runner.step(entries).shape[0] == 0                    # the prompts, eagerly, no logits wanted
    worst = decode_through_graphs(runner, seqs, tokens, fed, steps, folder, "wide")
    assert runner._graphs.replays == steps and list(runner._graphs.graphs) == [(1024, 256)]
    print(f"recorded steps of {n} sequences: worst {worst:.2f} of the bound")


def test_recorded_steps_at_real_layer_sizes_match_plain(tmp_path):
    """Two layers with the sizes of Qwen2.5-0.5B, decoded through recorded graphs: a batch of three (one padded
    row), a context that crosses 256 keys under way (another bucket: the chunks of keys are merged inside the
    output projection from there on), a request that joins late and one that leaves.  With up to 16 tokens the
    norms are folded into the products and the down product splits K between blocks."""
    import sprout_lm_amd as S
    from sprout_lm_amd.cli import PRESETS
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.weights import write_model_folder
    raw = dict(PRESETS["qwen2.5-0.5b"], num_hidden_layers=2)
    folder = str(tmp_path / "half_b")
    write_model_folder(folder, S.config_from_dict(raw), seed=9, dtype=torch.bfloat16, std=0.02)
    lengths = {"a": 250, "c": 5, "d": 100, "b": 300}
    tokens = {r: H.random_tokens(raw["vocab_size"], m + 24, 30 + i) for i, (r, m) in enumerate(lengths.items())}
    runner = ModelRunner.from_folder(folder, "bfloat16", block_size=16, num_blocks=64, max_sequences=4)
    seqs, fed = {}, {}

    def admit(r):
        seqs[r] = runner.cache.create()
        assert runner.cache.reserve(seqs[r], lengths[r])
        runner.step([StepEntry(seqs[r], tokens[r][:lengths[r]], [])])
        fed[r] = lengths[r]

    for r in "acd":
        admit(r)
    worst = decode_through_graphs(runner, seqs, tokens, fed, 10, folder, "three requests")       # a passes 256 keys
    assert set(runner._graphs.graphs) == {(4, 256), (4, 512)}
    admit("b")
    worst = max(worst, decode_through_graphs(runner, seqs, tokens, fed, 4, folder, "four requests"))
    seqs.pop("c").release()
    worst = max(worst, decode_through_graphs(runner, seqs, tokens, fed, 4, folder, "three requests again"))
    for s in seqs.values():
        s.release()
    assert runner.cache.free_pages() == [64]
    print(f"recorded steps at real layer sizes: worst {worst:.2f} of the bound")


def test_recorded_steps_of_forty_sequences_at_real_layer_sizes(tmp_path):
    """Between 17 and 64 sequences the decode kernels take the tokens in tiles along the grid (the q/k/v product
    with the norm folded in by 16, the accumulating products by 32) and the output head runs on the pipelined
    tiles: two layers with the sizes of Qwen2.5-0.5B, forty sequences at different positions (a recorded step of
    64 rows, 24 of them padding), every logit row against the plain side."""
    import sprout_lm_amd as S
    from sprout_lm_amd.cli import PRESETS
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.weights import write_model_folder
    raw = dict(PRESETS["qwen2.5-0.5b"], num_hidden_layers=2)
    folder = str(tmp_path / "half_b")
    write_model_folder(folder, S.config_from_dict(raw), seed=13, dtype=torch.bfloat16, std=0.02)
    n, steps = 40, 3
    rng = np.random.default_rng(8)
    tokens = {r: H.random_tokens(raw["vocab_size"], int(rng.integers(2, 40)) + steps, 200 + r) for r in range(n)}
    runner = ModelRunner.from_folder(folder, "bfloat16", block_size=16, num_blocks=4 * n, max_sequences=n)
    seqs = {r: runner.cache.create() for r in range(n)}
    fed = {r: len(tokens[r]) - steps for r in range(n)}
    entries = []
    for r in range(n):
        assert runner.cache.reserve(seqs[r], fed[r])
        entries.append(StepEntry(seqs[r], tokens[r][:fed[r]], []))
    assert runner.step(entries).shape[0] == 0
    worst = decode_through_graphs(runner, seqs, tokens, fed, steps, folder, "forty sequences")
    assert list(runner._graphs.graphs) == [(64, 256)]
    print(f"recorded steps of {n} sequences at real layer sizes: worst {worst:.2f} of the bound")


def fed_step(runner, seqs, tokens, fed, takes, folder, dtype, label, recorded=True):
    """One step in which request r brings its next `takes[r]` tokens and wants the logits of the last of them,
    through `step_recorded` (eagerly where that declines); every wanted row against the plain side.
    Returns (whether the step ran from a graph, worst error as a fraction of the bound)."""
    from sprout_lm_amd.engine import StepEntry
    entries = []
    for r, n in takes.items():
        assert runner.cache.reserve(seqs[r], fed[r] + n)
        entries.append(StepEntry(seqs[r], tokens[r][fed[r]:fed[r] + n], [n - 1]))
    logits = runner.step_recorded(entries) if recorded else None
    from_graph = logits is not None
    if logits is None:
        logits = runner.step(entries)
    got = logits.cpu().numpy()
    worst = 0.0
    for i, (r, n) in enumerate(takes.items()):
        fed[r] += n
        want = H.plain_logits(folder, dtype, tokens[r][:fed[r]], rows=[fed[r] - 1])[0]
        err = float(np.abs(got[i] - want).max()) / H.tolerance(dtype, want)
        worst = max(worst, err)
        assert err <= 1.0, f"{label}: request {r} up to position {fed[r] - 1}: {err:.2f} of the bound"
    return from_graph, worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_recorded_portions_match_plain(tmp_path, name, dtype):
    """Steps with portions of prompts are recorded when their shape comes a second time.  A prompt in equal
    portions (the last one shorter: another shape), then two requests that decode beside the portions of a
    third, which computes in the pages the first gave back; every step's wanted logits against the plain side,
    replay after replay, with eager steps of other shapes between them."""
    from sprout_lm_amd.engine import ModelRunner
    folder = H.make_model_folder(str(tmp_path), name)
    page = H.PAGE_SIZE[name]
    vocab = H.CONFIGS[name]["vocab_size"]
    tokens = {r: H.random_tokens(vocab, n, 500 + i) for i, (r, n) in enumerate(dict(a=127, b=40, c=47, d=118).items())}
    runner = ModelRunner.from_folder(folder, dtype, block_size=page, num_blocks=-(-127 // page) + 2 * -(-64 // page),
                                     max_sequences=4)
    seqs = {r: runner.cache.create() for r in "abc"}
    fed = dict.fromkeys("abcd", 0)
    ran, worst = [], 0.0
    for n in [24] * 5 + [7]:
        g, w = fed_step(runner, seqs, tokens, fed, {"a": n}, folder, dtype, "one prompt in portions")
        ran.append(g)
        worst = max(worst, w)
    assert ran == [False, True, True, True, True, False]         # recorded at the second sighting
    held = set(seqs["a"].blocks[0])
    seqs.pop("a").release()
    for r, n in (("b", 30), ("c", 41)):                           # two prompts, eagerly
        _, w = fed_step(runner, seqs, tokens, fed, {r: n}, folder, dtype, "whole prompt", recorded=False)
        worst = max(worst, w)
    seqs["d"] = runner.cache.create()
    ran = []
    for i in range(6):
        g, w = fed_step(runner, seqs, tokens, fed, {"b": 1, "d": 18, "c": 1}, folder, dtype, "decode beside a portion")
        ran.append(g)
        worst = max(worst, w)
        if i == 2:      # an eager step of another shape between replays, through the shared step context
            _, w = fed_step(runner, seqs, tokens, fed, {"d": 2}, folder, dtype, "two tokens", recorded=False)
            worst = max(worst, w)
    assert ran == [False] + [True] * 5
    assert held & set(seqs["d"].blocks[0]), "the late request got none of the pages that the first gave back"
    assert runner._graphs.portion_replays == 9
    for s in seqs.values():
        s.release()
    assert runner.cache.free_pages() == [runner.cache.num_blocks]
    print(f"recorded portions {name} {dtype}: worst {worst:.2f} of the bound")


def test_recorded_portions_at_real_layer_sizes_cross_a_context_bucket(tmp_path):
    """Two layers with the sizes of Qwen2.5-0.5B, a prompt of 512 tokens in portions of 64: the tiled products
    and the attention over tiles of queries, recorded.  The longest context a graph was recorded for is part of
    its key (256 keys, then 512): the step that first passes 256 keys runs eagerly and the next one is recorded
    anew."""
    import sprout_lm_amd as S
    from sprout_lm_amd.cli import PRESETS
    from sprout_lm_amd.engine import ModelRunner
    from sprout_lm_amd.weights import write_model_folder
    raw = dict(PRESETS["qwen2.5-0.5b"], num_hidden_layers=2)
    folder = str(tmp_path / "half_b")
    write_model_folder(folder, S.config_from_dict(raw), seed=9, dtype=torch.bfloat16, std=0.02)
    tokens = {"a": H.random_tokens(raw["vocab_size"], 512, 77)}
    runner = ModelRunner.from_folder(folder, "bfloat16", block_size=16, num_blocks=40, max_sequences=2)
    seqs, fed = {"a": runner.cache.create()}, {"a": 0}
    ran, worst = [], 0.0
    for _ in range(8):
        g, w = fed_step(runner, seqs, tokens, fed, {"a": 64}, folder, "bfloat16", "portions of 64")
        ran.append(g)
        worst = max(worst, w)
    assert ran == [False, True, True, True, False, True, True, True]
    assert set(runner._graphs.portion_graphs) == {(((64, 1),), 256), (((64, 1),), 512)}
    print(f"recorded portions at real layer sizes: worst {worst:.2f} of the bound")


def test_a_recorded_step_is_given_up_only_when_it_has_not_run_for_a_while(tmp_path):
    """Recording a step costs as much as dozens of steps.  With room for two recorded shapes, a third shape that
    keeps coming runs eagerly while both graphs are in use, and takes the place of the one that has not run for
    `keep_recent` steps; the logits are the plain implementation's whichever way a step runs."""
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    from sprout_lm_amd.engine.graphs import DecodeGraphs
    folder = H.make_model_folder(str(tmp_path), "A")
    vocab = H.CONFIGS["A"]["vocab_size"]
    runner = ModelRunner.from_folder(folder, "bfloat16", block_size=16, num_blocks=24, max_sequences=2)
    runner._graphs = DecodeGraphs(runner)
    runner._graphs.max_portion_graphs, runner._graphs.keep_recent = 2, 6
    tokens = {"a": H.random_tokens(vocab, 120, 900)}

    def run(n):
        """A fresh request fed its first `n` tokens as one step; whether that step ran from a graph."""
        seqs, fed = {"a": runner.cache.create()}, {"a": 0}
        from_graph, _ = fed_step(runner, seqs, tokens, fed, {"a": n}, folder, "bfloat16", f"{n} tokens")
        seqs["a"].release()
        return from_graph

    assert [run(5), run(5), run(7), run(7)] == [False, True, False, True]       # two shapes recorded
    assert [run(9), run(9), run(9)] == [False, False, False]                      # no room: both are in recent use
    assert [run(5) for _ in range(6)] == [True] * 6                               # the graph of 7 tokens grows old
    assert run(9) and set(k[0][0][0] for k in runner._graphs.portion_graphs) == {5, 9}
    assert not run(7)                                                             # its graph is gone; 5 and 9 are recent
