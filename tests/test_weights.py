"""Safetensors reading, sharded checkpoints, loader errors and the random-weights mode.

Reference: test/safetensors.test.ts:14-49, test/weight-files.test.ts:12-50.
"""
import json
import os
import struct

import numpy as np
import pytest
import torch

import sprout_lm_amd as S
from sprout_lm_amd.weights import (Checkpoint, SafetensorsError, SafetensorsFile, TensorSpec, WeightError,
                                   load_named_tensors, random_tensors, target_dtype, write_model_folder,
                                   write_safetensors)
from tests import helpers as H


def raw_file(path, header: dict, data: bytes):
    blob = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)) + blob + data)


def test_dtypes_are_read_as_stored(tmp_path):
    f32 = np.array([1.5, -2.25, 1e-40], dtype="<f4")                       # the last is subnormal
    bf16 = np.array([0x3FC0, 0xC010, 0x0001, 0x8000], dtype="<u2")         # 1.5, -2.25, subnormal, -0
    f16 = np.array([0x3E00, 0xC080, 0x0001, 0x7C00], dtype="<u2")          # 1.5, -2.25, 2^-24, inf
    header = {"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 12]},
              "b": {"dtype": "BF16", "shape": [2, 2], "data_offsets": [12, 20]},
              "c": {"dtype": "F16", "shape": [4], "data_offsets": [20, 28]},
              "__metadata__": {"format": "pt"}}
    path = tmp_path / "t.safetensors"
    raw_file(path, header, f32.tobytes() + bf16.tobytes() + f16.tobytes())
    f = SafetensorsFile(str(path))
    a, b, c = f.read("a"), f.read("b"), f.read("c")
    assert a.dtype == torch.float32 and np.array_equal(a.numpy(), f32)
    assert b.dtype == torch.bfloat16 and b.shape == (2, 2)
    assert b.float().flatten().tolist()[:2] == [1.5, -2.25] and b.float()[1, 0].item() == 2.0 ** -133
    assert c.dtype == torch.float16 and c.float().tolist() == [1.5, -2.25, 2.0 ** -24, float("inf")]
    f.close()


@pytest.mark.parametrize("case", ["truncated", "overlap", "gap", "range", "dtype", "size", "header"])
def test_malformed_files_are_refused(tmp_path, case):
    path = tmp_path / "bad.safetensors"
    data = bytes(16)
    entry = lambda b, e, dt="F32", shape=None: {"dtype": dt, "shape": shape or [(e - b) // 4], "data_offsets": [b, e]}
    if case == "truncated":
        path.write_bytes(b"\x10\x00\x00")
    elif case == "overlap":
        raw_file(path, {"a": entry(0, 8), "b": entry(4, 12)}, data[:12])
    elif case == "gap":
        raw_file(path, {"a": entry(0, 4), "b": entry(8, 16)}, data)
    elif case == "range":
        raw_file(path, {"a": entry(0, 32)}, data)
    elif case == "dtype":
        raw_file(path, {"a": entry(0, 16, "U8", [16])}, data)
    elif case == "size":
        raw_file(path, {"a": entry(0, 8)}, data)          # 8 bytes unaccounted for
    else:
        path.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(str(path))


def test_write_then_read_round_trip(tmp_path):
    tensors = {"w": torch.randn(3, 5).to(torch.bfloat16), "n": torch.randn(7), "t": torch.arange(6, dtype=torch.int32)}
    path = str(tmp_path / "m.safetensors")
    write_safetensors(path, tensors)
    f = SafetensorsFile(path)
    for name, t in tensors.items():
        assert torch.equal(f.read(name), t)
    f.close()
    from safetensors.torch import load_file     # an independent reader agrees
    for name, t in load_file(path).items():
        assert torch.equal(t, tensors[name])


def model_folder(tmp_path, name="A", storage=torch.bfloat16):
    return H.make_model_folder(str(tmp_path), name, storage)


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    folder = model_folder(tmp_path)
    cfg = S.load_config(folder)
    plan = S.build_model_plan(cfg)
    tensors = load_named_tensors(folder, plan.expected_tensors(), set(), torch.bfloat16, "cpu")
    assert set(tensors) == set(plan.expected_tensors())
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    norm = tensors["model.norm.weight"].float()
    assert abs(norm.mean().item() - 1.0) < 0.05          # norm weights are 1 + noise
    again = random_tensors(plan.expected_tensors(), H.SEEDS["A"], dtype=torch.bfloat16, std=H.WEIGHT_STD)
    assert all(torch.equal(again[k], tensors[k]) for k in tensors)      # same seed, same weights
    other = random_tensors(plan.expected_tensors(), H.SEEDS["A"] + 1, dtype=torch.bfloat16, std=H.WEIGHT_STD)
    assert not torch.equal(other["model.norm.weight"], tensors["model.norm.weight"])


def test_random_values_are_a_function_of_seed_name_and_index():
    """Element i of a tensor depends on (seed, name, i) alone: a piece drawn from the middle equals that piece of
    the whole, another name or seed gives other values, and the distribution has the asked deviation."""
    from sprout_lm_amd.weights.random_init import fill_numpy, key_for
    key = key_for(5, "model.layers.0.mlp.up_proj.weight")
    whole = fill_numpy(key, 300_000, 0.02 / 65536)
    assert np.array_equal(fill_numpy(key, 1000, 0.02 / 65536, first=123_457), whole[123_457:124_457])
    assert abs(whole.std() - 0.02) < 2e-4 and abs(whole.mean()) < 2e-4 and np.abs(whole).max() <= 0.12
    assert 0.04 < np.mean(np.abs(whole) > 0.04) < 0.05          # 4.55% of a normal distribution lie beyond two deviations
    assert not np.array_equal(fill_numpy(key_for(6, "model.layers.0.mlp.up_proj.weight"), 100, 1.0), whole[:100])
    assert key_for(5, "a") != key_for(5, "b")
    # the first values, pinned: the device kernel and any later rewrite must give these very numbers
    assert fill_numpy(key_for(1, "w"), 4, 1.0).tolist() == fill_numpy(key_for(1, "w"), 6, 1.0)[:4].tolist()
    ones = fill_numpy(key, 50, 0.02 / 65536, offset=1.0)
    assert np.array_equal(ones, whole[:50] + np.float32(1.0))


def test_a_tensor_stored_in_32_bit_stays_so(tmp_path):
    folder = model_folder(tmp_path, "A", torch.float32)
    plan = S.build_model_plan(S.load_config(folder))
    kept = load_named_tensors(folder, plan.expected_tensors(), set(), torch.bfloat16, "cpu")
    assert all(t.dtype == torch.float32 for t in kept.values())
    assert target_dtype(torch.bfloat16, "matrix", torch.bfloat16) == torch.bfloat16
    assert target_dtype(torch.float16, "matrix", torch.bfloat16) == torch.bfloat16
    assert target_dtype(torch.bfloat16, "vector", torch.float32) == torch.float32
    assert target_dtype(torch.int64, "int_table", torch.bfloat16) == torch.int32


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = model_folder(tmp_path)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.0.self_attn.k_proj.bias"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.1.mlp.up_proj.weight"] = torch.zeros(64, 128, dtype=torch.bfloat16)
    save_file(tensors, path)
    plan = S.build_model_plan(S.load_config(folder))
    with pytest.raises(WeightError) as info:
        load_named_tensors(folder, plan.expected_tensors(), set(plan.ignorable_tensors), torch.bfloat16, "cpu")
    error = info.value
    assert error.missing == ["model.layers.0.self_attn.k_proj.bias", "model.norm.weight"]
    assert error.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert [(n, tuple(w), tuple(g)) for n, w, g in error.wrong_shape] == [("model.layers.1.mlp.up_proj.weight", (128, 64), (64, 128))]
    text = str(error)
    for piece in ("missing tensors (2)", "k_proj.bias", "unexpected tensors (1)", "inv_freq", "expected [128, 64], got [64, 128]"):
        assert piece in text


def test_tensors_nobody_asked_for_are_left_unread_unless_strict(tmp_path):
    """The reference reads what it asks for and nothing else (src/safetensors.ts:70-83): a checkpoint that still
    ships a buffer such as rotary_emb.inv_freq loads; a strict load refuses it, naming it."""
    folder = model_folder(tmp_path)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(tensors, path)
    plan = S.build_model_plan(S.load_config(folder))
    notes = []
    loaded = load_named_tensors(folder, plan.expected_tensors(), set(plan.ignorable_tensors), torch.bfloat16, "cpu",
                                notes=notes)
    assert set(loaded) == set(plan.expected_tensors()) and len(notes) == 1 and "inv_freq" in notes[0]
    with pytest.raises(WeightError) as info:
        load_named_tensors(folder, plan.expected_tensors(), set(plan.ignorable_tensors), torch.bfloat16, "cpu", strict=True)
    assert info.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"] and not info.value.missing


def test_loaded_tensors_do_not_live_in_the_file(tmp_path):
    """Tensors go from the file's mapping to where they are kept without a host copy in between; a tensor kept
    on the host in its stored dtype must still be a copy (the file is closed, and may change, afterwards)."""
    folder = model_folder(tmp_path)
    plan = S.build_model_plan(S.load_config(folder))
    seen = {}
    loaded = load_named_tensors(folder, plan.expected_tensors(), set(), torch.bfloat16, "cpu",
                                before_read=lambda stored: seen.update(stored))
    assert set(seen) == set(plan.expected_tensors()) and set(seen.values()) == {torch.bfloat16}
    before = {k: v.clone() for k, v in loaded.items()}
    path = os.path.join(folder, "model.safetensors")
    size = os.path.getsize(path)
    with open(path, "r+b") as f:          # scribble over the data region
        f.seek(size // 2)
        f.write(b"\xff" * (size - size // 2))
    assert all(torch.equal(loaded[k].view(torch.int16), before[k].view(torch.int16)) for k in loaded)


def test_tied_checkpoint_may_ship_the_output_matrix(tmp_path):
    folder = model_folder(tmp_path)
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    save_file(tensors, path)
    plan = S.build_model_plan(S.load_config(folder))
    load_named_tensors(folder, plan.expected_tensors(), set(plan.ignorable_tensors), torch.float32, "cpu")


def test_sharded_checkpoint_equals_single_file(tmp_path):
    folder = model_folder(tmp_path, "B")
    single = Checkpoint(folder)
    names = sorted(single.names())
    shard_dir = tmp_path / "sharded"
    shard_dir.mkdir()
    halves = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    weight_map = {}
    for shard, members in halves.items():
        write_safetensors(str(shard_dir / shard), {n: single.read(n) for n in members})
        weight_map.update({n: shard for n in members})
    (shard_dir / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    (shard_dir / "config.json").write_text(open(os.path.join(folder, "config.json")).read())
    sharded = Checkpoint(str(shard_dir))
    assert sorted(sharded.names()) == names
    assert all(torch.equal(sharded.read(n), single.read(n)) for n in names)
    sharded.close(); single.close()
    # a tensor the index leaves out is missing; a shard name that climbs out of the folder is refused
    weight_map.pop(names[0])
    (shard_dir / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    plan = S.build_model_plan(S.load_config(str(shard_dir)))
    with pytest.raises(WeightError, match=names[0].replace(".", r"\.")):
        load_named_tensors(str(shard_dir), plan.expected_tensors(), set(), torch.float32, "cpu")
    # a name that the index maps to a shard which does not hold it
    bad = dict(weight_map)
    bad[names[0]] = "model-00002-of-00002.safetensors"
    (shard_dir / "model.safetensors.index.json").write_text(json.dumps({"weight_map": bad}))
    with pytest.raises(SafetensorsError, match="names 1 tensors that their shards do not hold: " + names[0].replace(".", r"\.")):
        Checkpoint(str(shard_dir))
    (shard_dir / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "../evil.safetensors"}}))
    with pytest.raises(SafetensorsError, match="shard filename"):
        Checkpoint(str(shard_dir))


def test_float16_tensors_widen_exactly_in_float32_and_are_noted_when_rounded_to_bfloat16(tmp_path):
    """float32 compute widens float16 exactly (reference: src/safetensors.ts:91-101); bfloat16 compute keeps 16-bit
    tensors in bfloat16, which loses three mantissa bits of a float16: the load says so."""
    from safetensors.torch import load_file, save_file
    folder = model_folder(tmp_path, "A")
    path = os.path.join(folder, "model.safetensors")
    tensors = {n: t.to(torch.float16) for n, t in load_file(path).items()}
    name = "model.layers.0.mlp.down_proj.weight"
    tensors[name][0, 0] = 1.0 + 2.0 ** -10          # a float16 that bfloat16 cannot hold
    save_file(tensors, path)
    plan = S.build_model_plan(S.load_config(folder))
    notes = []
    exact = load_named_tensors(folder, plan.expected_tensors(), set(), torch.float32, "cpu", notes=notes)
    assert not notes and exact[name][0, 0].item() == 1.0 + 2.0 ** -10
    rounded = load_named_tensors(folder, plan.expected_tensors(), set(), torch.bfloat16, "cpu", notes=notes)
    assert rounded[name].dtype == torch.bfloat16 and rounded[name][0, 0].item() == 1.0
    assert len(notes) == 1 and "stored in float16 were rounded to bfloat16" in notes[0] and str(len(tensors)) in notes[0]
