"""Engine against the plain implementation: each request alone and whole."""
import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("models"))
    return {name: H.make_model_folder(root, name) for name in H.CONFIGS}


def make_runner(folder, name, dtype, num_blocks=64, max_sequences=8):
    from sprout_lm_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, dtype, block_size=H.PAGE_SIZE[name], num_blocks=num_blocks,
                                   max_sequences=max_sequences)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_prompts_match_plain(folders, name, dtype):
    from sprout_lm_amd.engine import StepEntry
    runner = make_runner(folders[name], name, dtype)
    vocab = H.CONFIGS[name]["vocab_size"]
    for n, seed in ((1, 1), (5, 2), (17, 3), (33, 4), (70, 5)):
        tokens = H.random_tokens(vocab, n, seed)
        seq = runner.cache.create()
        assert runner.cache.reserve(seq, n)
        got = runner.step([StepEntry(seq, tokens, list(range(n)))]).cpu().numpy()
        seq.release()
        want = H.plain_logits(folders[name], dtype, tokens)
        err = np.abs(got - want).max()
        print(f"{name} {dtype} n={n}: max err {err:.3e} (scale {np.abs(want).max():.2f})")
        assert err <= H.tolerance(dtype, want)
    assert runner.cache.free_pages() == [64]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_far_positions_match_plain(folders, dtype):
    """Configuration C up to position 1,000, in portions and then token by token.  The error must not grow with
    the position: rotation angles of the float32 path are computed in float64 (a float32 angle is off by
    position * 6e-8, which at these positions is more than the whole bound)."""
    from sprout_lm_amd.engine import StepEntry
    name, n = "C", 1000
    runner = make_runner(folders[name], name, dtype, num_blocks=64)
    tokens = H.random_tokens(H.CONFIGS[name]["vocab_size"], n, 61)
    want = H.plain_logits(folders[name], dtype, tokens)
    seq = runner.cache.create()
    fed, worst_near, worst_far = 0, 0.0, 0.0
    for size in [300, 257, 300, 127] + [1] * 16:
        assert runner.cache.reserve(seq, fed + size)
        got = runner.step([StepEntry(seq, tokens[fed:fed + size], list(range(size)))]).cpu().numpy()
        for i in range(size):
            share = float(np.abs(got[i] - want[fed + i]).max()) / H.tolerance(dtype, want[fed + i])
            assert share <= 1.0, f"position {fed + i}: {share:.2f} of the bound"
            if fed + i < 200:
                worst_near = max(worst_near, share)
            elif fed + i >= 800:
                worst_far = max(worst_far, share)
        fed += size
    assert fed == n
    seq.release()
    print(f"{dtype}: worst share of the bound below position 200: {worst_near:.2f}, from 800 on: {worst_far:.2f}")
    assert worst_far <= max(2 * worst_near, 0.5)


def test_reference_fixture_logits_fp32(reference_fixture):
    """The reference's own fixture: logits computed by an independent library (test/qwen.test.ts:15-46).

    Head size 4 is outside what the bfloat16 kernels take; the float32 path takes any even head size.
    """
    import json, os
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    runner = ModelRunner.from_folder(reference_fixture, "float32", block_size=2, num_blocks=12, max_sequences=4)
    ref = json.load(open(os.path.join(reference_fixture, "reference.json")))
    for case in ref["cases"]:
        # a blocker takes a page first and gives it back later, so the request's second page is one that was
        # used before (and, in the first case, its pages are not in ascending order)
        blocker = runner.cache.create()
        assert runner.cache.reserve(blocker, 1)
        first = blocker.blocks[0][0]
        seq = runner.cache.create()
        history = list(case["tokens"])
        assert runner.cache.reserve(seq, 2)
        runner.step([StepEntry(seq, history[:2], [])])
        blocker.release()
        assert runner.cache.reserve(seq, len(history))
        logits = runner.step([StepEntry(seq, history[2:], [len(history) - 3])]).cpu().numpy()[0]
        assert seq.blocks[0][1] == first and seq.blocks[0][0] != first
        for step, name in enumerate(case["logits"]):
            want = np.fromfile(os.path.join(reference_fixture, name), dtype="<f4")
            assert np.abs(logits - want).max() < 1e-5      # the reference's GPU bound (test/cuda-device.integration.ts:38)
            assert int(np.argmax(logits)) == case["output"][step]
            if step + 1 < len(case["logits"]):
                assert runner.cache.reserve(seq, seq.length + 1)
                logits = runner.step([StepEntry(seq, [case["output"][step]], [0])]).cpu().numpy()[0]
        seq.release()
        assert runner.cache.free_pages() == [12]


def test_what_cannot_fit_is_refused_before_anything_is_allocated(folders):
    """Weights and cache pools are counted against the free device memory before the first tensor is read
    (reference: native/cuda-offload.cu:249-252): an absurd pool, or weights over their limit, are refused with a
    message that names the numbers, and no device memory has been taken."""
    import sprout_lm_amd as S
    from sprout_lm_amd.engine import ModelRunner
    from sprout_lm_amd.engine.memory import MemoryBudgetError
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    with pytest.raises(MemoryBudgetError, match=r"weights [\d,]+ MiB \+ cache pools [\d,]+ MiB \+ reserve 1,024 MiB = [\d,]+ MiB, free [\d,]+ MiB"):
        ModelRunner.from_folder(folders["C"], "bfloat16", block_size=16, num_blocks=2_000_000_000, max_sequences=4)
    with pytest.raises(MemoryBudgetError, match=r"Resident weight budget exceeded.*limit is 1 MiB"):
        ModelRunner.from_folder(folders["C"], "bfloat16", block_size=16, num_blocks=8, max_sequences=4, weight_limit_mib=1)
    with pytest.raises(MemoryBudgetError, match="reserve 400,000,000 MiB"):
        ModelRunner.from_config(S.config_from_dict(H.CONFIGS["A"]), 1, "float32", block_size=16, num_blocks=8,
                                max_sequences=4, reserve_mib=400_000_000)
    assert torch.cuda.memory_allocated() == before
    runner = ModelRunner.from_folder(folders["C"], "bfloat16", block_size=16, num_blocks=8, max_sequences=4, weight_limit_mib=2)
    assert runner.cache.free_pages() == [8]


def test_checkpoint_stored_in_32_bit_computed_in_bfloat16(tmp_path):
    """A tensor stored in 32-bit stays so: bfloat16 activations meet float32 weights (no rounding of the weights)."""
    import torch
    from sprout_lm_amd.engine import StepEntry
    from tests.plain import qwen2_plain as P
    folder = H.make_model_folder(str(tmp_path), "B", storage=torch.float32)
    runner = make_runner(folder, "B", "bfloat16")
    assert runner.parts.blocks[0].mixer.w_qkv.dtype == torch.float32
    cfg, w = P.load_folder(folder, "float32")              # the plain side keeps the float32 values too
    tokens = H.random_tokens(384, 45, 12)
    want = P.forward_logits(w, cfg, tokens, store=P.bf16_round)
    seq = runner.cache.create()
    assert runner.cache.reserve(seq, 45)
    got = runner.step([StepEntry(seq, tokens[:30], list(range(30)))]).cpu().numpy()
    got = np.concatenate([got, runner.step([StepEntry(seq, tokens[30:], list(range(15)))]).cpu().numpy()])
    assert np.abs(got - want).max() <= H.tolerance("bfloat16", want)
    rounded = P.forward_logits(P.load_folder(folder, "bfloat16")[1], cfg, tokens, store=P.bf16_round)
    assert np.abs(got - want).max() < np.abs(got - rounded).max()    # closer to the unrounded weights
