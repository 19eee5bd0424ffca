"""The model plan as data: what the parts of a layer keep, slot by slot, and who says whether prefixes are shared."""
import pytest

from sprout_lm_amd.cache import PagedKVSpec, StateSpec
from sprout_lm_amd.models.plan import LayerCall, LayerPlan, ModelPlan, PartPlan
from sprout_lm_amd.parts import Block, Mixer, register_part, registered_parts


def _register():
    if "plan_test_state" in registered_parts("mixer"):
        return

    @register_part("mixer", "plan_test_state")
    class Keeps(Mixer):
        def __init__(self, width, pieces=False):
            self.width, self.pieces = width, pieces

        def cache_spec(self):
            if self.pieces:
                return {"a": StateSpec((self.width,)), "b": PagedKVSpec(1, self.width)}
            return StateSpec((self.width,))

    @register_part("block", "plan_test_pair")
    class Pair(Block):
        def __init__(self, first, second):
            self.first, self.second = first, second

        def parts(self):
            return {"first": self.first, "second": self.second}


def plan_of(schedule, second=None, prefix_sharing=None):
    _register()
    attention = PartPlan("mixer", "attention", {"hidden": 32, "heads": 2, "kv_heads": 1, "head_dim": 16,
                                                "position": PartPlan("position", "none", {"head_dim": 16})}, "l0.attn.")
    second = second or PartPlan("mixer", "plan_test_state", {"width": 5}, "l0.keep.")
    norm = PartPlan("norm", "rmsnorm", {"size": 32, "eps": 1e-6}, "n.")
    return ModelPlan("PlanTest", None, 32, 50, 64, (0,), PartPlan("embedding", "token_embedding", {"vocab": 50, "hidden": 32}, "e."),
                     [LayerPlan("plan_test_pair", {"first": attention, "second": second})], schedule, norm,
                     PartPlan("head", "linear_head", {"vocab": 50, "hidden": 32, "tied": True}, "h."), prefix_sharing=prefix_sharing)


def test_a_call_names_the_slots_of_its_parts():
    parts = plan_of([LayerCall(0, {"first": 0, "second": 1}), LayerCall(0, {"first": 0, "second": 2}, writes={"first": False})]).instantiate()
    assert parts.call_slots == [{"first": (0, True), "second": (1, True)}, {"first": (0, False), "second": (2, True)}]
    assert parts.cache_slot_specs == [PagedKVSpec(1, 16), StateSpec((5,)), StateSpec((5,))]
    # a part that keeps several things by name: "part.piece"
    pieces = PartPlan("mixer", "plan_test_state", {"width": 8, "pieces": True}, "l0.keep.")
    parts = plan_of([LayerCall(0, {"first": 1, "second.a": 0, "second.b": 2})], second=pieces).instantiate()
    assert parts.cache_slot_specs == [StateSpec((8,)), PagedKVSpec(1, 16), PagedKVSpec(1, 8)]


def test_what_does_not_fit_is_refused_with_the_names():
    with pytest.raises(ValueError, match=r"one cache slot, but its parts ask for \['first', 'second'\]"):
        plan_of([LayerCall(0, 0)]).instantiate()
    with pytest.raises(ValueError, match=r"no part that keeps \['third'\]"):
        plan_of([LayerCall(0, {"first": 0, "third": 1})]).instantiate()
    with pytest.raises(ValueError, match="written by two calls"):
        plan_of([LayerCall(0, {"first": 0, "second": 1}), LayerCall(0, {"first": 0, "second": 2})]).instantiate()
    with pytest.raises(ValueError, match="numbered 0..n-1"):
        plan_of([LayerCall(0, {"first": 0, "second": 2})]).instantiate()
    with pytest.raises(ValueError, match="no call writes with the same shape"):
        plan_of([LayerCall(0, {"first": 0, "second": 1}), LayerCall(0, {"first": 1, "second": 2}, writes={"first": False})]).instantiate()


def test_the_plan_says_whether_prefixes_are_shared():
    """With per-request state of fixed size the default is no (a state is no function of pages); an architecture
    that can rebuild or snapshot its state says yes, and one without state may still say no."""
    slots = [LayerCall(0, {"first": 0, "second": 1})]
    assert plan_of(slots).instantiate().prefix_sharing is False
    assert plan_of(slots, prefix_sharing=True).instantiate().prefix_sharing is True
    assert plan_of([LayerCall(0, {"first": 0})]).instantiate().prefix_sharing is True
    assert plan_of([LayerCall(0, {"first": 0})], prefix_sharing=False).instantiate().prefix_sharing is False


def test_a_registered_step_array_is_laid_out_with_every_step():
    import numpy as np
    from sprout_lm_amd.cache import CacheManager
    from sprout_lm_amd.engine.batch import StepEntry, register_step_array, step_arrays, unregister_step_array
    cache = CacheManager([PagedKVSpec(1, 16)], block_size=4, num_blocks=8, max_sequences=2)
    a, b = cache.create(), cache.create()
    assert cache.reserve(a, 5) and cache.reserve(b, 9)
    cache.commit(b, 6)
    entries = [StepEntry(a, [1, 2, 3, 4, 5], [4]), StepEntry(b, [7, 8, 9], [])]
    register_step_array("plan_test_parity", "token", lambda layout: layout.positions % 2)
    register_step_array("plan_test_first", "sequence", lambda layout: layout.first_pos * 10)
    try:
        step = step_arrays(entries, cache)
        assert step.named("x:plan_test_parity").tolist() == [0, 1, 0, 1, 0, 0, 1, 0]
        assert step.named("x:plan_test_first").tolist() == [0, 60]
        register_step_array("plan_test_parity", "token", lambda layout: layout.positions[:3])
        with pytest.raises(ValueError, match="has 3 entries for 8 tokens"):
            step_arrays(entries, cache)
    finally:
        unregister_step_array("plan_test_parity")
        unregister_step_array("plan_test_first")
    assert not any(name.startswith("x:") for name in step_arrays(entries, cache).names)


def test_scratch_of_recorded_steps_is_freed_with_the_last_graph_that_used_it():
    """Recorded steps share scratch tensors that must never move while a graph holds their addresses; a tensor goes
    when the last graph that was handed it is given up, so shapes that come and go do not pile memory up."""
    import torch
    from sprout_lm_amd.engine.batch import KeptWorkspace, OwnedNames
    kept = KeptWorkspace("cpu")
    kept.owner = 1
    small = kept.get("residual", (4, 8), torch.float32)
    kept.owner = 2
    again = kept.get("residual", (2, 8), torch.float32)          # fits the tensor that graph 1 made: shared
    assert again.data_ptr() == small.data_ptr()
    large = kept.get("residual", (16, 8), torch.float32)         # a further tensor; the first one stays where it is
    assert large.data_ptr() != small.data_ptr() and kept.nbytes() == (32 + 128) * 4
    kept.release(1)                                              # graph 2 still uses both
    assert kept.nbytes() == (32 + 128) * 4
    kept.release(2)
    assert kept.nbytes() == 0
    # what a recorded step hands its caller is kept apart from the shared scratch
    own = OwnedNames(kept, ("logits",), "cpu")
    kept.owner = 3
    logits, scratch = own.get("logits", (2, 5), torch.float32), own.get("normed", (2, 5), torch.float32)
    assert kept.nbytes() == 40 and logits.data_ptr() != scratch.data_ptr()
    own.frozen = True
    with pytest.raises(RuntimeError, match="would grow while a graph is recorded"):
        own.get("logits", (3, 5), torch.float32)
    with pytest.raises(RuntimeError, match="would grow while a graph is recorded"):
        own.get("normed", (3, 5), torch.float32)
    own.frozen = False
