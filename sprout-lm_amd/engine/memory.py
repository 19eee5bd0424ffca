"""Device memory is counted before it is taken.

Reference: uploadMatrix (native/cuda-offload.cu:249-252) refuses a resident upload that would pass a
weight limit, or that would leave less than a reserve of free device memory.  Here the whole model is
sized at once, from the tensors its plan expects and from the cache manager's pools, before the first
tensor is read and before the pools are allocated; a model or pool that cannot fit is refused with one
message that names what is needed and what is there.
"""
from __future__ import annotations

from dataclasses import dataclass

from ..weights.loader import TensorSpec, target_dtype

MIB = 1024 * 1024
DEFAULT_RESERVE_MIB = 1024      # the reference's default reserve (src/cuda-offload.ts:48)


class MemoryBudgetError(RuntimeError):
    """The model's weights and cache pools do not fit the device memory that may be used."""


@dataclass(frozen=True)
class MemoryBudget:
    """weight_limit_mib: most device memory the weights may take (0: no limit of their own).
    reserve_mib: device memory that must stay free after weights and pools are allocated (workspace of the
    steps, recorded graphs, the runtime's own)."""

    weight_limit_mib: int = 0
    reserve_mib: int = DEFAULT_RESERVE_MIB

    def __post_init__(self):
        for name in ("weight_limit_mib", "reserve_mib"):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, int) or value < 0:
                raise ValueError(f"{name} must be a non-negative integer (MiB).")


def weight_bytes(expected: dict[str, TensorSpec], compute, stored: dict | None = None) -> int:
    """Device bytes of the tensors in `expected` under the engine's dtype policy (`target_dtype`).

    `stored`: name -> dtype the checkpoint holds the tensor in (absent: the compute dtype, as random
    weights are drawn)."""
    total = 0
    for name, spec in expected.items():
        kept = target_dtype((stored or {}).get(name, compute), spec.kind, compute)
        count = 1
        for n in spec.shape:
            count *= n
        total += count * kept.itemsize
    return total


def check_budget(weights: int, pools: int, free: int, budget: MemoryBudget, what: str = "model") -> None:
    """Raise MemoryBudgetError unless `weights` + `pools` bytes fit into `free` bytes with the reserve left."""
    limit = budget.weight_limit_mib * MIB
    if limit and weights > limit:
        raise MemoryBudgetError(
            f"Resident weight budget exceeded: the {what}'s weights take {weights / MIB:,.0f} MiB, the limit is "
            f"{budget.weight_limit_mib:,} MiB.")
    reserve = budget.reserve_mib * MIB
    if weights + pools + reserve > free:
        raise MemoryBudgetError(
            f"Insufficient free device memory for the {what}: weights {weights / MIB:,.0f} MiB + cache pools "
            f"{pools / MIB:,.0f} MiB + reserve {budget.reserve_mib:,} MiB = {(weights + pools + reserve) / MIB:,.0f} MiB, "
            f"free {free / MIB:,.0f} MiB.  Load fewer cache pages (num_blocks, block_size), a smaller dtype, or "
            f"lower the reserve.")


def free_device_bytes(device) -> int:
    """Bytes that an allocation could still get: what the driver reports free, plus what torch's allocator
    holds without using it."""
    import torch
    free, _ = torch.cuda.mem_get_info(device)
    return int(free) + int(torch.cuda.memory_reserved(device)) - int(torch.cuda.memory_allocated(device))
