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
    """One entry of the run order: run `layer`, its parts' caches in the slots `cache_slot` names.

    `cache_slot`: None (the layer keeps nothing), one slot number (for a layer in which exactly one part keeps
    something), or a mapping from what the layer's parts ask for to slot numbers: `{"mixer": 3}`, and, for a part
    whose `cache_spec` is itself a dict, `{"mixer.pages": 3, "mixer.tail": 4}`.  A layer may be called more than
    once (its weights are reused; give each call slots of its own), and a call with `writes` False reads slots
    that another call has written (`writes` may also be a mapping with the same keys).
    """

    layer: int
    cache_slot: int | dict | None
    writes: bool | dict = True


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
    # Whether requests may share the pages of a common prefix.  None: yes, unless some part keeps per-request
    # state of fixed size, which is no function of pages and would have to be rebuilt with them; an architecture
    # that knows better (a state it can snapshot at page edges, pages that depend on more than the tokens) says so.
    prefix_sharing: bool | None = None

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
        # What every call of the run order keeps where: per call {key: (slot, writes)}, key = a part's name in its
        # block, or "name.sub" where the part's cache_spec is a dict.
        self.call_slots: list[dict[str, tuple[int, bool]]] = []
        slots: dict[int, object] = {}
        for call in plan.schedule:
            if call.layer < 0 or call.layer >= len(self.blocks):
                raise ValueError(f"Run order names layer {call.layer}, but the model has {len(self.blocks)} layers.")
            needs = self.cache_needs(self.blocks[call.layer])
            if call.cache_slot is None:
                named = {}
            elif isinstance(call.cache_slot, dict):
                named = dict(call.cache_slot)
            else:
                if len(needs) != 1:
                    raise ValueError(f"Layer {call.layer} is given one cache slot, but its parts ask for "
                                     f"{sorted(needs) or 'none'}: name the slots by part.")
                named = {next(iter(needs)): call.cache_slot}
            unknown = sorted(set(named) - set(needs))
            if unknown:
                raise ValueError(f"Layer {call.layer} has no part that keeps {unknown}; its parts ask for {sorted(needs)}.")
            mine = {}
            for key, slot in named.items():
                writes = call.writes.get(key, True) if isinstance(call.writes, dict) else bool(call.writes)
                mine[key] = (slot, writes)
                if writes:
                    if slot in slots:
                        raise ValueError(f"Cache slot {slot} is written by two calls of the run order.")
                    slots[slot] = needs[key]
            self.call_slots.append(mine)
        for call, mine in zip(plan.schedule, self.call_slots):
            needs = self.cache_needs(self.blocks[call.layer])
            for key, (slot, writes) in mine.items():
                if not writes and slots.get(slot) != needs[key]:
                    raise ValueError(f"Layer {call.layer} reads cache slot {slot}, which no call writes with the "
                                     f"same shape.")
        if sorted(slots) != list(range(len(slots))):
            raise ValueError("Cache slots of the run order must be numbered 0..n-1 without gaps.")
        self.cache_slot_specs = [slots[i] for i in range(len(slots))]
        if plan.prefix_sharing is None:
            from ..cache.spec import StateSpec
            self.prefix_sharing = not any(isinstance(spec, StateSpec) for spec in self.cache_slot_specs)
        else:
            self.prefix_sharing = bool(plan.prefix_sharing)
        every = [part for _, part in self._named] + list(self.blocks)
        for part in list(every):
            every += part.subparts()
        self.graph_safe = all(getattr(part, "graph_safe", False) for part in every if part is not None)
        self.graph_safe_portions = self.graph_safe and all(getattr(part, "graph_safe_portions", False)
                                                           for part in every if part is not None)

    @staticmethod
    def cache_needs(block) -> dict:
        """What the parts of `block` keep between steps: {"part": spec} and {"part.sub": spec}."""
        needs = {}
        for name, part in block.parts().items():
            spec = part.cache_spec()
            if isinstance(spec, dict):
                needs.update({f"{name}.{sub}": one for sub, one in spec.items()})
            elif spec is not None:
                needs[name] = spec
        return needs

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
        return sum(part.cache_elements_per_token() for block in self._calls() for part in block.parts().values()) * element_size

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
