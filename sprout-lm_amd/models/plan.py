"""A model as data: which parts make up each layer, what their tensors are called, and the order
in which layers run.  Architectures produce a ModelPlan from their configuration; nothing else in
the engine knows an architecture by name."""
from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.base import Part, make_part
from ..weights.loader import TensorSpec


@dataclass
class PartPlan:
    """One part: registry category and kind, constructor parameters, and the checkpoint prefix of its
    tensors.  A parameter may itself be a PartPlan (a position encoding inside a mixer)."""

    category: str
    kind: str
    params: dict = field(default_factory=dict)
    prefix: str = ""

    def make(self) -> Part:
        params = {k: (v.make() if isinstance(v, PartPlan) else v) for k, v in self.params.items()}
        return make_part(self.category, self.kind, **params)


@dataclass
class LayerPlan:
    """A block kind and the parts it arranges (constructor argument name -> part)."""

    block: str
    parts: dict[str, PartPlan]


@dataclass
class LayerCall:
    """One entry of the run order: run `layer` with cache slot `cache_slot`.

    A layer may be called more than once (its weights are reused; give each call a slot of its
    own), and a call with writes False reads a slot that another call has written.
    """

    layer: int
    cache_slot: int | None
    writes: bool = True


@dataclass
class ModelPlan:
    architecture: str
    config: object
    hidden_size: int
    vocab_size: int
    max_positions: int
    eos_token_ids: tuple[int, ...]
    embedding: PartPlan
    layers: list[LayerPlan]
    schedule: list[LayerCall]
    final_norm: PartPlan
    head: PartPlan
    ignorable_tensors: frozenset = frozenset()

    def instantiate(self) -> "ModelParts":
        return ModelParts(self)

    def expected_tensors(self) -> dict[str, TensorSpec]:
        return self.instantiate().expected_tensors()


class ModelParts:
    """The part objects of a plan, with the full names of their tensors."""

    def __init__(self, plan: ModelPlan):
        self.plan = plan
        self.embedding = plan.embedding.make()
        self.final_norm = plan.final_norm.make()
        self.head = plan.head.make()
        self.blocks = []
        self._named: list[tuple[str, Part]] = [(plan.embedding.prefix, self.embedding),
                                               (plan.final_norm.prefix, self.final_norm),
                                               (plan.head.prefix, self.head)]
        for layer in plan.layers:
            made = {name: part.make() for name, part in layer.parts.items()}
            self.blocks.append(make_part("block", layer.block, **made))
            self._named.extend((layer.parts[name].prefix, made[name]) for name in layer.parts)
        slots: dict[int, object] = {}
        for call in plan.schedule:
            if call.layer < 0 or call.layer >= len(self.blocks):
                raise ValueError(f"Run order names layer {call.layer}, but the model has {len(self.blocks)} layers.")
            spec = self.blocks[call.layer].mixer.cache_spec()
            if call.cache_slot is None:
                continue
            if call.writes:
                if call.cache_slot in slots:
                    raise ValueError(f"Cache slot {call.cache_slot} is written by two calls of the run order.")
                slots[call.cache_slot] = spec
        for call in plan.schedule:
            if call.cache_slot is not None and not call.writes:
                spec = self.blocks[call.layer].mixer.cache_spec()
                if slots.get(call.cache_slot) != spec:
                    raise ValueError(f"Layer {call.layer} reads cache slot {call.cache_slot}, which no call writes "
                                     f"with the same shape.")
        if sorted(slots) != list(range(len(slots))):
            raise ValueError("Cache slots of the run order must be numbered 0..n-1 without gaps.")
        self.cache_slot_specs = [slots[i] for i in range(len(slots))]
        every = [part for _, part in self._named] + list(self.blocks)
        every += [getattr(b.mixer, "position", None) for b in self.blocks if hasattr(b, "mixer")]
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in every if part is not None)
        self.graph_safe_portions = self.graph_safe and all(getattr(part, "graph_safe_portions", False)
                                                           for part in every if part is not None)

    # ------------------------------------------------------------------ what a step costs, summed over the parts
    def _calls(self):
        """(block, cache slot) of every entry of the run order: a layer that runs twice counts twice."""
        return [self.blocks[call.layer] for call in self.plan.schedule]

    def weight_bytes(self, element_size: int) -> int:
        """Bytes of weights that one step reads: every tensor of every part that runs, once."""
        seen, total = set(), 0
        parts = [self.final_norm, self.head] + [p for block in self._calls() for p in block.parts().values()]
        for part in parts:
            if id(part) not in seen:       # a layer that runs twice reads its weights twice, but from the caches
                seen.add(id(part))
                total += part.weight_elements()
        return total * element_size

    def cache_bytes_per_context_token(self, element_size: int) -> int:
        """Cache bytes that one decoded token reads per token of its context, over all calls of the run order."""
        return sum(block.mixer.cache_elements_per_token() for block in self._calls() if hasattr(block, "mixer")) * element_size

    def flops(self, tokens: int, pairs: int, logit_rows: int) -> float:
        """Matrix-product operations of a step of `tokens` tokens with `pairs` (query, key) pairs in every
        mixer and `logit_rows` rows of logits."""
        total = self.head.flops(logit_rows)
        for block in self._calls():
            total += sum(part.flops(tokens, pairs) for part in block.parts().values())
        return total

    def expected_tensors(self) -> dict[str, TensorSpec]:
        out = {}
        for prefix, part in self._named:
            for local, spec in part.tensors().items():
                out[prefix + local] = spec
        return out

    def bind(self, tensors: dict, device, dtype) -> None:
        """Hand every part its tensors.  They are taken out of `tensors` as they go: a part that joins
        several of them into one (q, k and v; gate and up) then holds the only copy, and the separate ones
        are freed layer by layer instead of all at the end."""
        again: dict = {}        # tensors that two parts name (weights shared by name)
        names = [prefix + local for prefix, part in self._named for local in part.tensors()]
        shared = {n for n in names if names.count(n) > 1}
        for prefix, part in self._named:
            mine = {}
            for local in part.tensors():
                name = prefix + local
                mine[local] = again[name] if name in again else tensors.pop(name)
                if name in shared:
                    again[name] = mine[local]
            part.bind(mine)
            part.prepare(device, dtype)
        if getattr(self.head, "tied", False):
            self.head.tie(self.embedding.w["weight"])
